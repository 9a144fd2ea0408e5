"""Every executable copy direction exactly once, chained: the idea of the reference's on-hardware
test test/python/hybm/data_op_all_path_test.py (graph of valid (source kind, destination kind)
pairs walked along an Eulerian path, MD5 of the first and the last block compared), for the
kinds one rank on one GPU has: local host, local device, pool host, pool device.  Driven through
the hybm_* layer with explicit directions, once with single copies and once with batches."""

import ctypes
import hashlib

import numpy as np
import pytest

from memfabric_hybrid_amd import native
from tests import gpu_util
from tests.oracle_lib import np_ptr

MIB = 1 << 20
POOL = 64 * MIB
BLOCK = 3 * MIB + 4093  # odd on purpose

KINDS = ["LH", "LD", "GH", "GD"]
EDGES = [(s, d) for s in KINDS for d in KINDS if not (s[0] == "L" and d[0] == "L")]


def eulerian_path(start):
    """Hierholzer, as in the reference's resolver: consume edges greedily, emit nodes on backtrack."""
    edges = list(EDGES)
    stack, path = [start], []
    while stack:
        top = stack[-1]
        nxt = next((e for e in edges if e[0] == top), None)
        if nxt:
            edges.remove(nxt)
            stack.append(nxt[1])
        else:
            path.append(stack.pop())
    assert not edges
    return path[::-1]


@pytest.fixture(scope="module")
def entity(lib):
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    opts = native.HybmOptions()
    opts.bmType = 1          # HYBM_TYPE_HOST_INITIATE
    opts.memType = native.HYBM_MEM_TYPE_DEVICE | native.HYBM_MEM_TYPE_HOST
    opts.bmDataOpType = 2    # HYBM_DOP_TYPE_SDMA: the intra-node engine
    opts.rankCount, opts.rankId, opts.devId = 1, 0, 0
    opts.maxHBMSize = opts.deviceVASpace = POOL
    opts.maxDRAMSize = opts.hostVASpace = POOL
    opts.scene = 1
    opts.dramShmFd = -1
    e = lib.hybm_create_entity(200, ctypes.byref(opts), 0)
    assert e, native.last_error()
    assert lib.hybm_reserve_mem_space(e, 0) == 0
    assert lib.hybm_alloc_local_memory(e, native.HYBM_MEM_TYPE_DEVICE, POOL, 0)
    assert lib.hybm_alloc_local_memory(e, native.HYBM_MEM_TYPE_HOST, POOL, 0)
    yield e
    lib.hybm_destroy_entity(e, 0)
    lib.hybm_uninit()


def test_path_covers_every_direction_once():
    path = eulerian_path("LH")
    walked = list(zip(path, path[1:]))
    assert sorted(walked) == sorted(EDGES) and len(walked) == 12
    assert path[0] == path[-1] == "LH"


@pytest.mark.gpu
@pytest.mark.parametrize("batched", [False, True])
@pytest.mark.parametrize("pinned_local_host", [False, True])
def test_walk_all_directions(lib, entity, oracle, batched, pinned_local_host):
    gd = lib.hybm_get_memory_ptr(entity, native.HYBM_MEM_TYPE_DEVICE)
    gh = lib.hybm_get_memory_ptr(entity, native.HYBM_MEM_TYPE_HOST)
    slots = 8
    ld = gpu_util.DeviceBuffer(lib, slots * (BLOCK + 64))
    if pinned_local_host:
        lh_buf = gpu_util.PinnedBuffer(lib, slots * (BLOCK + 64))
        lh_arr, lh_base = lh_buf.array, lh_buf.ptr
    else:
        lh_arr = np.zeros(slots * (BLOCK + 64), dtype=np.uint8)
        lh_base = np_ptr(lh_arr)
    base = {"LH": lh_base, "LD": ld.ptr, "GH": gh, "GD": gd}
    visits = {k: 0 for k in KINDS}

    def fresh(kind):
        off = visits[kind] * (BLOCK + 64) + visits[kind] % 7   # shifting misalignment
        visits[kind] += 1
        return base[kind] + off

    try:
        first = np.empty(BLOCK, dtype=np.uint8)
        oracle.orc_fill_random(np_ptr(first), BLOCK, 0xE1)
        path = eulerian_path("LH")
        cur = fresh("LH")
        ctypes.memmove(cur, np_ptr(first), BLOCK)
        digest_first = hashlib.md5(first.tobytes()).hexdigest()
        for src_kind, dst_kind in zip(path, path[1:]):
            dst = fresh(dst_kind)
            direction = native.HYBM_DIR[f"{src_kind}2{dst_kind}"]
            if batched:
                cuts = [0, 5, 4096, MIB + 3, BLOCK]
                srcs = native.ptr_array([cur + a for a in cuts[:-1]])
                dsts = native.ptr_array([dst + a for a in cuts[:-1]])
                lens = native.u64_array([b - a for a, b in zip(cuts, cuts[1:])])
                params = native.BatchCopyParams(srcs, dsts, lens, len(cuts) - 1)
                ret = lib.hybm_data_batch_copy(entity, ctypes.byref(params), direction, None, 0)
            else:
                params = native.HybmCopyParams(cur, dst, BLOCK)
                ret = lib.hybm_data_copy(entity, ctypes.byref(params), direction, None, 0)
            assert ret == 0, (src_kind, dst_kind, native.last_error())
            cur = dst
        assert path[-1] == "LH"
        last = np.empty(BLOCK, dtype=np.uint8)
        ctypes.memmove(np_ptr(last), cur, BLOCK)
        assert hashlib.md5(last.tobytes()).hexdigest() == digest_first
        assert np.array_equal(last, first)
    finally:
        ld.free()
        if pinned_local_host:
            lh_buf.free()


@pytest.mark.gpu
def test_auto_direction_and_caller_stream(lib, entity, oracle):
    """AUTO infers pool/pool and local/pool directions; a copy on a caller's stream is ordered
    after work the caller queued there before (a fill kernel produces the source)."""
    gd = lib.hybm_get_memory_ptr(entity, native.HYBM_MEM_TYPE_DEVICE)
    gh = lib.hybm_get_memory_ptr(entity, native.HYBM_MEM_TYPE_HOST)
    n = 16 * MIB
    stream = lib.mfrt_stream_create()
    local = gpu_util.DeviceBuffer(lib, n)
    try:
        assert lib.mfrt_memset(gd, 0, 2 * n) == 0
        for _ in range(3):  # producer and consumer back to back on the caller's stream
            assert native.yardstick().mf_probe_hbm(1, local.ptr, None, n, stream) == 0   # fills with the word 0x5A
            params = native.HybmCopyParams(local.ptr, gd + n, n)
            assert lib.hybm_data_copy(entity, ctypes.byref(params), native.HYBM_DIR["AUTO"], stream,
                                      native.ASYNC_COPY_FLAG) == 0, native.last_error()
        assert lib.mfrt_stream_sync(stream) == 0
        got = np.empty(n, dtype=np.uint8)
        assert lib.mfrt_memcpy(np_ptr(got), gd + n, n) == 0
        assert np.all(got.view(np.uint32) == 0x5A)
        # pool device -> pool host by AUTO
        params = native.HybmCopyParams(gd + n, gh + 4096, n)
        assert lib.hybm_data_copy(entity, ctypes.byref(params), native.HYBM_DIR["AUTO"], None, 0) == 0
        assert np.all(gpu_util.host_view(gh + 4096, n).view(np.uint32) == 0x5A)
        # two private addresses cannot be inferred
        other = gpu_util.DeviceBuffer(lib, 4096)
        params = native.HybmCopyParams(local.ptr, other.ptr, 4096)
        assert lib.hybm_data_copy(entity, ctypes.byref(params), native.HYBM_DIR["AUTO"], None, 0) == native.BM_INVALID_PARAM
        other.free()
    finally:
        local.free()
        lib.mfrt_stream_destroy(stream)
