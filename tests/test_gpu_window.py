"""Mapped device windows on the GPU (the default mode): the device window is reserved address
space, local allocations map HBM into it piece by piece (the job of the reference's
HybmDevLegacySegment, src/hybm/csrc/mm/hybm_dev_legacy_segment.cpp:123-181), and copies inside the
mapped prefix are byte-exact against the oracle, also across the seam between two mappings."""

import ctypes
import os

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu

MIB = 1 << 20


@pytest.fixture()
def mapped_entity(lib):
    old = os.environ.pop("MF_HIP_GVA_WINDOW", None)     # read when the address space is reserved
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    opts = native.HybmOptions()
    opts.bmType = 1
    opts.memType = native.HYBM_MEM_TYPE_DEVICE
    opts.bmDataOpType = 2
    opts.rankCount, opts.rankId, opts.devId = 1, 0, 0
    opts.maxHBMSize = 4096 * MIB                  # the window: far more than is ever mapped
    opts.deviceVASpace = 256 * MIB
    opts.scene = 1
    opts.dramShmFd = -1
    e = lib.hybm_create_entity(210, ctypes.byref(opts), 0)
    assert e, native.last_error()
    assert lib.hybm_reserve_mem_space(e, 0) == 0, native.last_error()
    yield e
    lib.hybm_destroy_entity(e, 0)
    lib.hybm_uninit()
    if old is not None:
        os.environ["MF_HIP_GVA_WINDOW"] = old


def test_copies_inside_and_across_mappings(lib, oracle, mapped_entity):
    e = mapped_entity
    base = lib.hybm_get_memory_ptr(e, native.HYBM_MEM_TYPE_DEVICE)
    assert base
    first = lib.hybm_alloc_local_memory(e, native.HYBM_MEM_TYPE_DEVICE, 96 * MIB, 0)
    second = lib.hybm_alloc_local_memory(e, native.HYBM_MEM_TYPE_DEVICE, 160 * MIB, 0)
    assert first and second, native.last_error()
    assert lib.hybm_get_slice_va(e, first) == base and lib.hybm_get_slice_va(e, second) == base + 96 * MIB
    pool = 256 * MIB
    data = np.empty(pool, dtype=np.uint8)
    oracle.orc_fill_random(np_ptr(data), pool, 0x3A9)
    pinned = gpu_util.PinnedBuffer(lib, pool)
    try:
        pinned.array[:] = data
        # host -> pool in one copy that spans the seam between the two mappings
        params = native.HybmCopyParams(pinned.ptr, base, pool)
        assert lib.hybm_data_copy(e, ctypes.byref(params), native.HYBM_DIR["LH2GD"], None, 0) == 0, native.last_error()
        # KV batch inside the pool; some segments straddle the seam by construction of the offsets
        src, dst, lens = workloads.kv_batch(0x3AA, pool)
        seam = 96 * MIB
        dst[0] = seam - 4096                              # a 128 KiB segment written across the seam ...
        src[1] = seam + 64 * MIB - 8192                   # ... and one read from well inside the second mapping
        want = data.copy()
        order = [i for i in range(len(lens)) if i not in (0, 1)]
        assert not _overlaps(src[1], dst[1], lens[1], src[:1], dst[:1], lens[:1])
        keep = [0, 1] + [i for i in order if not (_overlaps(src[i], dst[i], lens[i], src[:2], dst[:2], lens[:2]))]
        src, dst, lens = src[keep], dst[keep], lens[keep]
        gpu_util.oracle_batch(oracle, data, want, src, dst, lens)
        batch = native.BatchCopyParams(native.ptr_array((base + src).tolist()), native.ptr_array((base + dst).tolist()),
                                       native.u64_array(lens.tolist()), len(lens))
        assert lib.hybm_data_batch_copy(e, ctypes.byref(batch), native.HYBM_DIR["GD2GD"], None, 0) == 0, native.last_error()
        # a single copy whose source straddles the seam
        params = native.HybmCopyParams(base + seam - MIB - 5, base + 200 * MIB + 3, 2 * MIB + 11)
        assert lib.hybm_data_copy(e, ctypes.byref(params), native.HYBM_DIR["GD2GD"], None, 0) == 0, native.last_error()
        want[200 * MIB + 3:200 * MIB + 3 + 2 * MIB + 11] = want[seam - MIB - 5:seam + MIB + 6].copy()
        got = np.empty(pool, dtype=np.uint8)
        assert lib.mfrt_memcpy(np_ptr(got), base, pool) == 0      # plain runtime copy out of the mapped window
        assert np.array_equal(got, want)
        # one byte past the mapped prefix is refused on the host, nothing is launched
        launches = lib.mf_xcopy_launch_count()
        params = native.HybmCopyParams(pinned.ptr, base + pool - 4096, 8192)
        assert lib.hybm_data_copy(e, ctypes.byref(params), native.HYBM_DIR["LH2GD"], None, 0) == native.BM_INVALID_PARAM
        assert lib.mf_xcopy_launch_count() == launches
        # memory goes back from the top; the window then ends at the first mapping again
        assert lib.hybm_free_local_memory(e, second, 1, 0) == 0
        params = native.HybmCopyParams(pinned.ptr, base + 96 * MIB, 4096)
        assert lib.hybm_data_copy(e, ctypes.byref(params), native.HYBM_DIR["LH2GD"], None, 0) == native.BM_INVALID_PARAM
        params = native.HybmCopyParams(base, pinned.ptr, 96 * MIB)
        pinned.array[:96 * MIB] = 0
        assert lib.hybm_data_copy(e, ctypes.byref(params), native.HYBM_DIR["GD2LH"], None, 0) == 0
        assert np.array_equal(pinned.array[:96 * MIB], want[:96 * MIB])
    finally:
        pinned.free()


def _overlaps(s, d, n, srcs, dsts, lens):
    """True when segment (s, d, n) reads or writes bytes the given segments write, or writes bytes
    they read: the batch must stay free of overlap after two of its segments were moved."""
    for s2, d2, n2 in zip(srcs, dsts, lens):
        for a, an, b, bn in ((d, n, d2, n2), (d, n, s2, n2), (s, n, d2, n2)):
            if int(a) < int(b) + int(bn) and int(b) < int(a) + int(an):
                return True
    return False
