"""GPU parity on the remaining benchmark shapes: strided 2-D copies, the paged KV
gather/scatter and the TP8 -> TP4 weight re-layout.  All byte movement: bit-exact."""

import ctypes

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu

MIB = 1 << 20


@pytest.fixture(scope="module")
def gpu(lib):
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    yield lib
    lib.hybm_uninit()


def _rand(oracle, n, seed):
    a = np.empty(n, dtype=np.uint8)
    oracle.orc_fill_random(np_ptr(a), n, seed)
    return a


def _copy2d(gpu, rects, route=native.ROUTE_HBM):
    descs = (native.Copy2dDesc * len(rects))()
    for i, r in enumerate(rects):
        descs[i] = native.Copy2dDesc(*[int(v) for v in r])
    ret = gpu.mf_xcopy_2d_batch(descs, len(rects), route, None)
    assert ret == 0, native.last_error()
    assert gpu.mfrt_device_sync() == 0


@pytest.mark.parametrize("width,height,spitch,dpitch,soff,doff", [
    (896, 3584, 896, 1792, 0, 0),          # the o_proj merge geometry
    (4736, 300, 4736, 9472, 0, 4736),      # the down_proj merge geometry, right half
    (16, 1000, 48, 32, 16, 0),             # one unit per row
    (32768, 5, 40000 - 40000 % 16, 65536, 0, 0),  # rows wider than a chunk
    (2 * MIB + 16, 3, 2 * MIB + 48, 2 * MIB + 16, 32, 0),   # rows wider than 1 MiB: 131 073 units, beyond a 16-bit division trick
    (1048592, 2, 1048592, 1048608, 0, 16),  # 65 537 units per row
    (100, 77, 160, 300, 5, 11),            # nothing aligned: falls back to one segment per row
    (48, 1, 48, 48, 0, 0),
])
def test_2d_copy_matches_the_oracle(gpu, oracle, width, height, spitch, dpitch, soff, doff):
    src_bytes = soff + spitch * height + 64
    dst_bytes = doff + dpitch * height + 64
    src = _rand(oracle, src_bytes, width)
    sbuf = gpu_util.DeviceBuffer(gpu, src_bytes)
    dbuf = gpu_util.DeviceBuffer(gpu, dst_bytes)
    try:
        sbuf.upload(src)
        dbuf.fill(0x5C)
        _copy2d(gpu, [(sbuf.ptr + soff, dbuf.ptr + doff, width, height, spitch, dpitch)])
        got = dbuf.download()
    finally:
        sbuf.free()
        dbuf.free()
    expect = np.full(dst_bytes, 0x5C, dtype=np.uint8)
    oracle.orc_copy_2d(np_ptr(expect) + doff, dpitch, np_ptr(src) + soff, spitch, width, height)
    assert np.array_equal(got, expect)


def test_2d_batch_of_many_rectangles(gpu, oracle):
    """150 rectangles (more than one launch holds), mixed widths, tiled into disjoint destinations."""
    rng = np.random.default_rng(21)
    src = _rand(oracle, 8 * MIB, 21)
    sbuf = gpu_util.DeviceBuffer(gpu, 8 * MIB)
    dbuf = gpu_util.DeviceBuffer(gpu, 64 * MIB)
    rects, model = [], []
    cursor = 0
    for i in range(150):
        width = int(rng.choice([16, 64, 896, 1000, 4736, 20000]))
        height = int(rng.integers(1, 60))
        spitch = (width + int(rng.integers(0, 4)) * 16 + 15) // 16 * 16 if width % 16 == 0 else width + 7
        dpitch = spitch + 32
        soff = int(rng.integers(0, 8 * MIB - spitch * height - 16)) // 16 * 16
        rects.append((sbuf.ptr + soff, dbuf.ptr + cursor, width, height, spitch, dpitch))
        model.append((soff, cursor, width, height, spitch, dpitch))
        cursor += (dpitch * height + 255) // 256 * 256
    assert cursor <= 64 * MIB
    try:
        sbuf.upload(src)
        dbuf.fill(0)
        _copy2d(gpu, rects)
        got = dbuf.download(0, cursor)
    finally:
        sbuf.free()
        dbuf.free()
    expect = np.zeros(cursor, dtype=np.uint8)
    for soff, doff, width, height, spitch, dpitch in model:
        oracle.orc_copy_2d(np_ptr(expect) + doff, dpitch, np_ptr(src) + soff, spitch, width, height)
    assert np.array_equal(got, expect)


def test_2d_batch_in_read_and_write_windows(gpu, oracle):
    """A launch that moves more than 512 MiB between device addresses takes the windowed rectangle kernel (chunks of
    1024 units of the payload taken row-major): two mates of the down_proj geometry, rows of one unit, rows narrower
    and wider than a chunk, a row count that leaves a partial last chunk.  Compared with the oracle byte for byte,
    gaps between the rows included."""
    shapes = [(4736, 57001, 4736, 9472), (4736, 57001, 4736, 9472), (16, 3001, 32, 48), (48, 1000, 64, 80),
              (40000, 51, 40016, 40032), (16384, 33, 16384, 16400), (16400, 7, 16416, 16400)]
    src_at, dst_at, sbytes, dbytes = [], [], 0, 0
    for i, (w, h, sp, dp) in enumerate(shapes):
        src_at.append(sbytes)
        sbytes += sp * h + 16
        if i == 1:
            dst_at.append(dst_at[0] + shapes[0][0])      # side by side with the first
            continue
        dst_at.append(dbytes)
        dbytes += dp * h + 16
    assert sum(w * h for w, h, _, _ in shapes) > 512 * MIB
    src = _rand(oracle, sbytes, 77)
    sbuf = gpu_util.DeviceBuffer(gpu, sbytes)
    dbuf = gpu_util.DeviceBuffer(gpu, dbytes)
    try:
        sbuf.upload(src)
        dbuf.fill(0x5C)
        _copy2d(gpu, [(sbuf.ptr + src_at[i], dbuf.ptr + dst_at[i], w, h, sp, dp) for i, (w, h, sp, dp) in enumerate(shapes)])
        got = dbuf.download()
    finally:
        sbuf.free()
        dbuf.free()
    expect = np.full(dbytes, 0x5C, dtype=np.uint8)
    for i, (w, h, sp, dp) in enumerate(shapes):
        oracle.orc_copy_2d(np_ptr(expect) + dst_at[i], dp, np_ptr(src) + src_at[i], sp, w, h)
    assert np.array_equal(got, expect)


def test_2d_argument_errors(gpu):
    d = (native.Copy2dDesc * 1)(native.Copy2dDesc(0x1000, 0x2000, 64, 4, 32, 64))
    assert gpu.mf_xcopy_2d_batch(d, 1, 0, None) == native.BM_INVALID_PARAM      # width > source pitch
    assert gpu.mf_xcopy_2d_batch(None, 1, 0, None) == native.BM_INVALID_PARAM
    assert gpu.mf_xcopy_2d_batch(d, 0, 0, None) == 0


def test_paged_kv_gather_then_scatter_is_identity(gpu, oracle):
    """4096 distinct 32 KiB pages gathered into a contiguous buffer and scattered back to fresh
    locations; gather compared with the oracle, scatter(gather(x)) compared with x."""
    page = 32768
    pool_pages = 16384                       # 512 MiB pool at test size
    count = 4096
    pool = _rand(oracle, pool_pages * page, 0xC3)
    ids = workloads.page_ids(0xC3, pool_pages, count)
    pbuf = gpu_util.DeviceBuffer(gpu, pool_pages * page)
    cbuf = gpu_util.DeviceBuffer(gpu, count * page)
    qbuf = gpu_util.DeviceBuffer(gpu, pool_pages * page)
    try:
        pbuf.upload(pool)
        qbuf.fill(0)
        contiguous = np.arange(count, dtype=np.uint64) * page
        gpu_util.xcopy(gpu, pbuf.ptr + ids * page, cbuf.ptr + contiguous, [page] * count, native.ROUTE_HBM)
        got = cbuf.download()
        expect = np.zeros(count * page, dtype=np.uint8)
        gpu_util.oracle_batch(oracle, pool, expect, ids * page, contiguous, [page] * count)
        assert np.array_equal(got, expect)
        gpu_util.xcopy(gpu, cbuf.ptr + contiguous, qbuf.ptr + ids * page, [page] * count, native.ROUTE_HBM)
        back = qbuf.download()
        touched = np.zeros(pool_pages, dtype=bool)
        touched[ids.astype(np.int64)] = True
        back_pages = back.reshape(pool_pages, page)
        assert np.array_equal(back_pages[touched], pool.reshape(pool_pages, page)[touched])
        assert not back_pages[~touched].any()
    finally:
        pbuf.free()
        cbuf.free()
        qbuf.free()


def _run_reshard(gpu, tensors, layers, s_pool):
    _, _, s_bytes, d_bytes = workloads.reshard_layout(tensors, layers)
    sbuf = gpu_util.DeviceBuffer(gpu, s_bytes)
    dbuf = gpu_util.DeviceBuffer(gpu, d_bytes)
    try:
        sbuf.upload(s_pool.view(np.uint8))
        dbuf.fill(0xEE)
        segments, rects = workloads.reshard_plan(tensors, layers, sbuf.ptr, dbuf.ptr)
        gpu_util.xcopy(gpu, [s for s, _, _ in segments], [d for _, d, _ in segments], [n for _, _, n in segments],
                       native.ROUTE_HBM, sync=False)
        _copy2d(gpu, rects)
        return dbuf.download().view(np.uint16)
    finally:
        sbuf.free()
        dbuf.free()


def test_reshard_tp8_to_tp4_small_model(gpu):
    """A scaled-down decoder (same structure): the GPU re-layout of the TP8 storage equals the
    TP4 shards cut directly out of the full tensors."""
    tensors = workloads.reshard_tensors(hidden=256, ffn=1280, kv_heads=4, head_dim=32)
    layers = 3
    rng = np.random.default_rng(0xC5)
    full = {(l, name): rng.integers(0, 65536, (out, cols), dtype=np.uint16)
            for l in range(layers) for name, out, cols, _ in tensors}
    s_pool, d_pool = workloads.reshard_reference(tensors, layers, full)
    got = _run_reshard(gpu, tensors, layers, s_pool)
    assert np.array_equal(got, d_pool)


def test_reshard_full_size_layer(gpu):
    """One layer at the real shape (hidden 3584, FFN 18944, 4 KV heads): 466 MB in, 452 MB out."""
    tensors = workloads.reshard_tensors()
    rng = np.random.default_rng(0xC5)
    full = {(0, name): rng.integers(0, 65536, (out, cols), dtype=np.uint16) for name, out, cols, _ in tensors}
    s_pool, d_pool = workloads.reshard_reference(tensors, 1, full)
    got = _run_reshard(gpu, tensors, 1, s_pool)
    assert np.array_equal(got, d_pool)
