"""The copy plugin driven the way the reference drives it: its own loader
(src/hybm/csrc/under_api/dl_hybm_copy_extend.cpp:25-86 of the reference, compiled as it is into
oracle/_ref) finds libmf_hybm_copy_extend.so through MEMFABRIC_HYBRID_EXTEND_LIB_PATH, opens it with
dlopen(RTLD_NOW | RTLD_NODELETE), wants both symbols, and HostDataOpSDMA-style calls go through its
thunks (dl_hybm_copy_extend.h:29-51)."""

import os
import subprocess

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from tests import gpu_util
from tests.oracle_lib import np_ptr

ENV = "MEMFABRIC_HYBRID_EXTEND_LIB_PATH"
BM_OK, BM_ERROR, BM_DL_FUNCTION_FAILED, BM_UNDER_API_UNLOAD = 0, -1, -6, -8
MIB = 1 << 20


@pytest.fixture
def loader(ref):
    saved = os.environ.pop(ENV, None)
    ref.ref_extend_cleanup()
    yield ref
    ref.ref_extend_cleanup()
    if saved is None:
        os.environ.pop(ENV, None)
    else:
        os.environ[ENV] = saved


def test_loader_finds_the_plugin_only_where_the_environment_points(loader, tmp_path):
    assert loader.ref_extend_try_load() == BM_ERROR                      # variable not set
    assert loader.ref_extend_batch_copy(None, 0, None, 32, None) == BM_UNDER_API_UNLOAD
    os.environ[ENV] = str(tmp_path / "nowhere")
    assert loader.ref_extend_try_load() == BM_ERROR                      # not a directory
    # a library of the right name with only one of the two symbols is opened and dropped again
    half = tmp_path / "half"
    half.mkdir()
    src = half / "half.c"
    src.write_text("void hybm_copy_extend(void *a, void *b, unsigned long c, unsigned d, void *e) {}\n")
    subprocess.run(["gcc", "-shared", "-fPIC", "-o", str(half / "libmf_hybm_copy_extend.so"), str(src)], check=True)
    os.environ[ENV] = str(half)
    assert loader.ref_extend_try_load() == BM_DL_FUNCTION_FAILED
    assert loader.ref_extend_copy(None, None, 0, 32, None) == BM_UNDER_API_UNLOAD
    # the product's plugin satisfies the loader
    os.environ[ENV] = native.LIB_DIR
    assert loader.ref_extend_try_load() == BM_OK
    assert loader.ref_extend_try_load() == BM_OK                         # idempotent


@pytest.mark.gpu
def test_copies_through_the_reference_loader(loader, lib, oracle):
    """hybm_batch_copy_extend as HostDataOpSDMA::BatchCopyExtend issues it
    (src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:504-543 of the reference): a pinned
    parameter slot of {src, dst, len} triples, the slot's completion word, HYBM_EXTEND_CONCURRENT = 32."""
    os.environ[ENV] = native.LIB_DIR
    assert loader.ref_extend_try_load() == BM_OK
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    n = 32 * MIB
    pool = gpu_util.DeviceBuffer(lib, 2 * n)
    slot = gpu_util.PinnedBuffer(lib, 16384 * 24 + 64)
    stream = lib.mfrt_stream_create()
    try:
        init = np.empty(2 * n, dtype=np.uint8)
        oracle.orc_fill_random(np_ptr(init), 2 * n, 0xE7)
        pool.upload(init)
        expect = init.copy()
        for count, seed in ((122, 1), (5000, 2)):
            src, dst, lens = workloads.ragged_batch(seed, 2 * n, count, max_len=3000 if count > 200 else 60000)
            triples = np.empty((count, 3), dtype=np.uint64)
            triples[:, 0], triples[:, 1], triples[:, 2] = pool.ptr + src, pool.ptr + dst, lens
            raw = triples.view(np.uint8).reshape(-1)
            slot.array[:len(raw)] = raw
            word = slot.array[16384 * 24:16384 * 24 + 8].view(np.uint64)
            word[0] = 0
            assert loader.ref_extend_batch_copy(slot.ptr, count, slot.ptr + 16384 * 24, 32, stream) == BM_OK
            assert lib.mfrt_stream_sync(stream) == 0
            assert word[0] == 32                                          # the slot may be refilled
            gpu_util.oracle_batch(oracle, expect.copy(), expect, src, dst, lens)
            assert np.array_equal(pool.download(), expect)
        # the single-copy symbol, odd alignment on both sides
        assert loader.ref_extend_copy(pool.ptr + 5, pool.ptr + n + 3, 7 * MIB + 1, 32, stream) == BM_OK
        assert lib.mfrt_stream_sync(stream) == 0
        expect[n + 3:n + 3 + 7 * MIB + 1] = expect[5:5 + 7 * MIB + 1].copy()
        assert np.array_equal(pool.download(), expect)
    finally:
        lib.mfrt_stream_destroy(stream)
        slot.free()
        pool.free()
        lib.hybm_uninit()
