"""Size-independent properties at the full sizes of the benchmark configurations that the byte-for-byte
oracle comparisons (run at sizes the CPU finishes in seconds) do not reach: 1 GiB and 2 GiB single
copies host -> device -> device -> host through smem_bm_copy, and the paged KV gather / scatter on a
40 GiB pool.  Sources are built from one random block XORed with a per-block constant, so every
64 MiB of a large buffer differs and a piece that lands at a wrong offset cannot go unnoticed."""

import ctypes

import numpy as np
import pytest

from memfabric_hybrid_amd import bm, native, workloads
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu

MIB = 1 << 20
GIB = 1 << 30
GUARD = 2 * MIB


def _pattern_block(oracle):
    block = np.empty(64 * MIB, dtype=np.uint8)
    oracle.orc_fill_random(np_ptr(block), len(block), 0xF5)
    return block


def _fill_pattern(view, block):
    for i in range(0, len(view), len(block)):
        m = min(len(block), len(view) - i)
        np.bitwise_xor(block[:m], np.uint8((i // len(block) * 29 + 3) & 0xFF), out=view[i:i + m])


def _same_as_pattern(view, block):
    for i in range(0, len(view), len(block)):
        m = min(len(block), len(view) - i)
        if not np.array_equal(view[i:i + m], block[:m] ^ np.uint8((i // len(block) * 29 + 3) & 0xFF)):
            return False
    return True


@pytest.fixture(scope="module")
def pool(lib):
    assert bm.initialize("tcp://127.0.0.1:0", 1, 0) == 0, native.last_error()
    p = bm.create(7, 2 * (2 * GIB + GUARD) + GUARD, 2 * (2 * GIB + GUARD) + GUARD)
    yield p
    p.destroy()
    bm.uninitialize()


@pytest.mark.parametrize("nbytes", [GIB, 2 * GIB], ids=["1GiB", "2GiB"])
def test_single_copies_at_full_size_host_device_device_host(pool, lib, oracle, nbytes):
    """smem_bm_copy of 1 GiB / 2 GiB: pinned host pool -> HBM pool (host link), HBM -> HBM, HBM ->
    pinned host pool (host link); what arrives back equals what left, and the guard bytes round
    every destination are untouched."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    span = 2 * GIB + GUARD
    host_all = gpu_util.host_view(host, 2 * span + GUARD)
    block = _pattern_block(oracle)
    src_off, back_off = GUARD, span + GUARD                  # two host regions, guards in front, between and behind
    dev_a, dev_b = GUARD, span + GUARD
    host_all[:] = 0xA5
    _fill_pattern(host_all[src_off:src_off + nbytes], block)
    assert lib.mfrt_memset(dev, 0x5A, 2 * span + GUARD) == 0
    g2g = bm.BmCopyType.G2G
    assert pool.copy_data(host + src_off, dev + dev_a, nbytes, g2g) == 0, native.last_error()          # H2D
    assert pool.copy_data(dev + dev_a, dev + dev_b, nbytes, g2g) == 0, native.last_error()              # D2D
    assert pool.copy_data(dev + dev_b, host + back_off, nbytes, g2g) == 0, native.last_error()          # D2H
    assert _same_as_pattern(host_all[back_off:back_off + nbytes], block)
    assert np.all(host_all[back_off - GUARD:back_off] == 0xA5)
    assert np.all(host_all[back_off + nbytes:back_off + nbytes + GUARD] == 0xA5)
    edge = np.empty(GUARD, dtype=np.uint8)
    for at in (dev_a - GUARD, dev_a + nbytes, dev_b - GUARD, dev_b + nbytes):
        if at + GUARD <= 2 * span + GUARD and not (dev_a <= at < dev_a + nbytes) and not (dev_b <= at < dev_b + nbytes):
            assert lib.mfrt_memcpy(np_ptr(edge), dev + at, GUARD) == 0
            assert np.all(edge == 0x5A), at
    # idempotence: the same device -> device copy once more changes nothing
    assert pool.copy_data(dev + dev_a, dev + dev_b, nbytes, g2g) == 0, native.last_error()
    assert pool.copy_data(dev + dev_b, host + back_off, nbytes, g2g) == 0, native.last_error()
    assert _same_as_pattern(host_all[back_off:back_off + nbytes], block)


@pytest.mark.parametrize("agree", [True, False], ids=["same-modulo-16", "apart-modulo-16"])
@pytest.mark.parametrize("pieces", [7, 200], ids=["7-pieces", "200-pieces"])
@pytest.mark.parametrize("rate", [-1, 7400000, 0], ids=["default-windows", "short-periods", "no-windows"])
def test_ragged_batch_above_one_gib_in_read_and_write_windows(pool, lib, oracle, rate, pieces, agree):
    """A device-to-device batch of 1 GiB and more goes through the kernel that alternates between read and
    write windows.  Seven pieces of about 170 MB, or 200 of about 6 MB (a table that the engine cuts into
    launches of 128 segments), with odd lengths at odd source and destination addresses (partial first and
    last chunks, head and tail bytes), with the default period, with a period too short for the waves to
    keep up (they then proceed late; the result must not depend on timing) and with the form switched off:
    what comes back equals the same slices cut on the CPU, and the bytes between and round the destinations
    are untouched.  Sources and destinations either agree modulo 16 (the batch then takes the windows) or do not
    (the engine then leaves the windows out, whatever the rate)."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    span = 2 * GIB + GUARD
    host_all = gpu_util.host_view(host, 2 * span + GUARD)
    block = _pattern_block(oracle)
    total = GIB + 256 * MIB
    _fill_pattern(host_all[GUARD:GUARD + total], block)
    g2g = bm.BmCopyType.G2G
    assert pool.copy_data(host + GUARD, dev + GUARD, total, g2g) == 0, native.last_error()
    assert lib.mfrt_memset(dev + span, 0x5A, span) == 0
    rng = np.random.default_rng(21)
    each = (GIB + 100 * MIB) // pieces
    lens = rng.integers(each - each // 20, each + each // 25, pieces) | 1  # odd lengths
    gaps = rng.integers(1, 4096, pieces) | 1
    src = GUARD + np.cumsum(lens + gaps) - lens                            # odd addresses
    dst = span + GUARD + np.cumsum(lens + 2 * gaps + 17) - lens
    if agree:
        dst = dst + ((src - dst) % 16)
    else:
        dst = dst + ((src - dst) % 16 == 0)
    assert bool(np.all((src - dst) % 16 == 0)) == agree and bool(np.any((src - dst) % 16 == 0)) == agree
    assert int(lens.sum()) >= GIB and int(src[-1] + lens[-1]) <= GUARD + total
    assert int(dst[-1] + lens[-1]) + GUARD <= 2 * span + GUARD
    try:
        if rate >= 0:
            assert lib.mf_xcopy_windows(rate) == 0
        assert pool.copy_data_batch((dev + src).tolist(), (dev + dst).tolist(), lens.tolist(), len(lens), g2g, 0) == 0, \
            native.last_error()
    finally:
        assert lib.mf_xcopy_windows(1) == 0        # the library's own choice again
    assert lib.mf_xcopy_windows(999) != 0
    lo, hi = int(dst[0]) - GUARD, int(dst[-1] + lens[-1]) + GUARD
    back = span + GUARD                                                    # the second host region
    assert hi - lo <= span
    assert pool.copy_data(dev + lo, host + back, hi - lo, g2g) == 0, native.last_error()
    got = host_all[back:back + hi - lo]
    cursor = lo
    for s_off, d_off, n in zip(src.tolist(), dst.tolist(), lens.tolist()):
        assert np.all(got[cursor - lo:d_off - lo] == 0x5A), d_off          # the gap in front of the piece
        assert np.array_equal(got[d_off - lo:d_off - lo + n], host_all[s_off:s_off + n]), d_off
        cursor = d_off + n
    assert np.all(got[cursor - lo:] == 0x5A)


@pytest.mark.parametrize("layout", ["on-cache-lines", "between-cache-lines", "apart-modulo-16"])
@pytest.mark.parametrize("total_mib", [130, 200, 300], ids=["130MiB", "200MiB", "300MiB"])
def test_batches_of_some_hundred_mib_in_windows_whose_last_period_is_full(pool, lib, oracle, total_mib, layout):
    """Device-to-device batches of 130 to 300 MiB in 37 ragged segments: sizes whose chunks do not fill a whole number
    of periods on 4096 waves, so the launch runs on fewer waves with every period full.  Segments on cache lines
    (the higher window rate), between cache lines (the general rate) and with sources apart from their destinations
    modulo 16 (no windows): what arrives equals the same slices cut on the CPU, the gaps between destinations stay."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    span = 2 * GIB + GUARD
    host_all = gpu_util.host_view(host, 2 * span + GUARD)
    block = _pattern_block(oracle)
    total = total_mib * MIB
    room = total + 64 * MIB
    _fill_pattern(host_all[GUARD:GUARD + room], block)
    g2g = bm.BmCopyType.G2G
    assert pool.copy_data(host + GUARD, dev + GUARD, room, g2g) == 0, native.last_error()
    assert lib.mfrt_memset(dev + span, 0x5A, room + 2 * GUARD) == 0
    rng = np.random.default_rng(total_mib)
    pieces = 37
    each = total // pieces
    unit = 128 if layout == "on-cache-lines" else 16
    lens = rng.integers(each - each // 10, each + each // 10, pieces)
    lens = lens // unit * unit if layout == "on-cache-lines" else (lens | 1)
    gaps = rng.integers(1, 64, pieces) * unit
    src = GUARD + np.cumsum(lens + gaps) - lens
    src = (src + unit - 1) // unit * unit
    dst = span + GUARD + np.cumsum(lens + 3 * gaps) - lens
    dst = (dst + unit - 1) // unit * unit
    if layout == "between-cache-lines":
        src, dst = src + 16, dst + 48
    elif layout == "apart-modulo-16":
        src, dst = src + 5, dst + 9
    assert int(src[-1] + lens[-1]) <= GUARD + room and int(dst[-1] + lens[-1]) + GUARD <= span + 2 * GUARD + room
    assert np.all(src[1:] >= src[:-1] + lens[:-1]) and np.all(dst[1:] >= dst[:-1] + lens[:-1])
    assert pool.copy_data_batch((dev + src).tolist(), (dev + dst).tolist(), lens.tolist(), len(lens), g2g, 0) == 0, \
        native.last_error()
    lo, hi = int(dst[0]) - GUARD, int(dst[-1] + lens[-1]) + GUARD
    back = span + GUARD
    assert pool.copy_data(dev + lo, host + back, hi - lo, g2g) == 0, native.last_error()
    got = host_all[back:back + hi - lo]
    cursor = lo
    for s_off, d_off, n in zip(src.tolist(), dst.tolist(), lens.tolist()):
        assert np.all(got[cursor - lo:d_off - lo] == 0x5A), d_off
        assert np.array_equal(got[d_off - lo:d_off - lo + n], host_all[s_off:s_off + n]), d_off
        cursor = d_off + n
    assert np.all(got[cursor - lo:] == 0x5A)


def test_table_of_segments_on_cache_lines_is_cut_into_windowed_launches(pool, lib, oracle):
    """300 segments of about 1.5 MiB on cache lines, shuffled: more than the kernel-argument form holds, so the engine cuts
    the table into launches of 128 segments (192 MiB each, in read and write windows; the last 44 segments without).  Every
    segment arrives, the gaps between destinations stay, and mf_xcopy_windows(1) has brought the library's own rates back."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    span = 2 * GIB + GUARD
    host_all = gpu_util.host_view(host, 2 * span + GUARD)
    block = _pattern_block(oracle)
    count, slot = 300, 2 * MIB
    room = count * slot
    _fill_pattern(host_all[GUARD:GUARD + room], block)
    g2g = bm.BmCopyType.G2G
    assert pool.copy_data(host + GUARD, dev + GUARD, room, g2g) == 0, native.last_error()
    assert lib.mfrt_memset(dev + span, 0x5A, room + 2 * GUARD) == 0
    rng = np.random.default_rng(300)
    lens = (rng.integers(MIB + MIB // 4, 2 * MIB - 4096, count) // 128 * 128).astype(np.int64)
    order = rng.permutation(count)
    src = GUARD + order * slot + rng.integers(0, 16, count) * 128
    dst = span + GUARD + np.arange(count) * slot + rng.integers(0, 16, count) * 128
    assert lib.mf_xcopy_windows(1) == 0
    before = lib.mf_xcopy_launch_count()
    assert pool.copy_data_batch((dev + src).tolist(), (dev + dst).tolist(), lens.tolist(), count, g2g, 0) == 0, native.last_error()
    if _window_rate(lib) != 0:
        assert lib.mf_xcopy_launch_count() - before == 3
    lo, hi = int(dst[0]) - GUARD, int(dst[-1] + lens[-1]) + GUARD
    back = span + GUARD
    assert pool.copy_data(dev + lo, host + back, hi - lo, g2g) == 0, native.last_error()
    got = host_all[back:back + hi - lo]
    cursor = lo
    for s_off, d_off, n in zip(src.tolist(), dst.tolist(), lens.tolist()):
        assert np.all(got[cursor - lo:d_off - lo] == 0x5A), d_off
        assert np.array_equal(got[d_off - lo:d_off - lo + n], host_all[s_off:s_off + n]), d_off
        cursor = d_off + n
    assert np.all(got[cursor - lo:] == 0x5A)


def test_one_segment_beyond_four_gib_goes_out_in_windowed_launches(lib, oracle):
    """One device-to-device segment of 5 GiB + 4 MiB + 777 bytes (its length does not fit 32 bits) from an odd source
    address to an odd destination address: the engine cuts it into windowed launches of about 512 MiB.  Every byte
    arrives (each 64 MiB of the source differs from the others, so a piece at a wrong offset shows), and the bytes
    in front of and behind the destination stay as they were."""
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    nbytes = 5 * GIB + 4 * MIB + 777
    room = nbytes + 2 * GUARD
    src = lib.mfrt_alloc_device(room)
    dst = lib.mfrt_alloc_device(room)
    if not src or not dst:
        for p in (src, dst):
            if p:
                lib.mfrt_free_device(p)
        lib.hybm_uninit()
        pytest.skip("two device allocations of 5 GiB are not available on this GPU right now")
    try:
        block = _pattern_block(oracle)
        s_at, d_at = src + GUARD + 5, dst + GUARD + 21        # the same modulo 16: the copy takes the windows
        piece = np.empty(len(block), dtype=np.uint8)
        for i in range(0, nbytes, len(block)):
            m = min(len(block), nbytes - i)
            np.bitwise_xor(block[:m], np.uint8((i // len(block) * 29 + 3) & 0xFF), out=piece[:m])
            assert lib.mfrt_memcpy(s_at + i, np_ptr(piece), m) == 0
        assert lib.mfrt_memset(dst, 0x5A, room) == 0
        assert lib.mfrt_device_sync() == 0
        before = lib.mf_xcopy_launch_count()
        gpu_util.xcopy(lib, [s_at], [d_at], [nbytes], native.ROUTE_HBM)
        launches = lib.mf_xcopy_launch_count() - before
        if _window_rate(lib) != 0:      # the start-up check may have found that windows gain nothing on this GPU
            assert launches == nbytes // (512 * MIB), launches
        for i in range(0, nbytes, len(block)):
            m = min(len(block), nbytes - i)
            assert lib.mfrt_memcpy(np_ptr(piece), d_at + i, m) == 0
            assert np.array_equal(piece[:m], block[:m] ^ np.uint8((i // len(block) * 29 + 3) & 0xFF)), i
        edge = np.empty(GUARD + 21, dtype=np.uint8)
        assert lib.mfrt_memcpy(np_ptr(edge), dst, GUARD + 21) == 0
        assert np.all(edge == 0x5A)
        assert lib.mfrt_memcpy(np_ptr(edge), d_at + nbytes, GUARD - 21) == 0
        assert np.all(edge[:GUARD - 21] == 0x5A)
    finally:
        lib.mfrt_free_device(src)
        lib.mfrt_free_device(dst)
        lib.hybm_uninit()


def _window_rate(lib):
    rate = ctypes.c_uint32(0)
    lib.mf_xcopy_calibration(None, None, ctypes.byref(rate), None, None, None)
    return rate.value


def test_paged_gather_and_scatter_on_a_40_gib_pool(lib, oracle):
    """4096 distinct 32 KiB pages sampled from a 40 GiB HBM pool (offsets far beyond 32 bits):
    gather equals the sampled pages in order; scattering them to 4096 other pages and gathering
    those returns the same bytes; pages next to the targets are untouched."""
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    page, count = 32768, 4096
    pool_bytes = 40 * GIB
    pool = lib.mfrt_alloc_device(pool_bytes)
    if not pool:
        lib.hybm_uninit()
        pytest.skip("a 40 GiB device allocation is not available on this GPU right now")
    flat = gpu_util.DeviceBuffer(lib, count * page)
    again = gpu_util.DeviceBuffer(lib, count * page)
    try:
        total_pages = pool_bytes // page
        picks = workloads.page_ids(0xC3, total_pages, 2 * count)
        ids, fresh = picks[:count], picks[count:]
        assert int(ids.max()) * page > (1 << 35)             # the sample really reaches the far end
        pages = np.empty((count, page), dtype=np.uint8)
        oracle.orc_fill_random(np_ptr(pages), pages.size, 0xC3)
        filler = np.full(page, 0x77, dtype=np.uint8)
        for i in range(count):                               # only the sampled pages and the scatter targets are initialised
            assert lib.mfrt_memcpy(pool + int(ids[i]) * page, pages[i].ctypes.data, page) == 0
            assert lib.mfrt_memcpy(pool + int(fresh[i]) * page, filler.ctypes.data, page) == 0
        lanes = np.arange(count, dtype=np.uint64) * page
        gpu_util.xcopy(lib, pool + ids * page, flat.ptr + lanes, [page] * count, native.ROUTE_HBM)
        assert np.array_equal(flat.download().reshape(count, page), pages)
        gpu_util.xcopy(lib, flat.ptr + lanes, pool + fresh * page, [page] * count, native.ROUTE_HBM)
        gpu_util.xcopy(lib, pool + fresh * page, again.ptr + lanes, [page] * count, native.ROUTE_HBM)
        assert np.array_equal(again.download().reshape(count, page), pages)
        # the originals are still in place (the scatter went elsewhere)
        probe = np.empty(page, dtype=np.uint8)
        for i in range(0, count, 257):
            assert lib.mfrt_memcpy(np_ptr(probe), pool + int(ids[i]) * page, page) == 0
            assert np.array_equal(probe, pages[i])
    finally:
        flat.free()
        again.free()
        lib.mfrt_free_device(pool)
        lib.hybm_uninit()
