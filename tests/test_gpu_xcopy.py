"""GPU parity of the xcopy path: every test drives the HIP kernels through the C
ABI and compares bytes with the CPU oracle on the same seeded inputs (bit-exact:
the path is byte movement)."""

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
    lib.mf_xcopy_tune(0, 0, 0)
    lib.hybm_uninit()


def _random_bytes(oracle, nbytes, seed):
    a = np.empty(nbytes, dtype=np.uint8)
    oracle.orc_fill_random(np_ptr(a), nbytes, seed)
    return a


def _check_d2d(gpu, oracle, pool_bytes, src_off, dst_off, lens, seed, units=0):
    gpu.mf_xcopy_tune(units, 16 if units else 0, 0)
    init = _random_bytes(oracle, pool_bytes, seed)
    buf = gpu_util.DeviceBuffer(gpu, pool_bytes)
    try:
        buf.upload(init)
        gpu_util.xcopy(gpu, buf.ptr + src_off, buf.ptr + dst_off, lens, native.ROUTE_HBM)
        got = buf.download()
    finally:
        buf.free()
    expect = init.copy()
    gpu_util.oracle_batch(oracle, init, expect, src_off, dst_off, lens)
    assert np.array_equal(got, expect)


def test_runtime_reports_the_gpu(gpu):
    assert gpu.mfrt_is_initialised() == 1
    assert gpu.mfrt_cu_count() >= 64
    p = gpu.mfrt_alloc_device(4096)
    h = gpu.mfrt_alloc_host(4096)
    stack = np.zeros(16, dtype=np.uint8)
    assert gpu.mfrt_pointer_kind(p) == native.PTR_DEVICE
    assert gpu.mfrt_pointer_kind(h) == native.PTR_PINNED_HOST
    assert gpu.mfrt_pointer_kind(np_ptr(stack)) == native.PTR_PAGEABLE
    gpu.mfrt_free_device(p)
    gpu.mfrt_free_host(h)


@pytest.mark.parametrize("units", [0, 256, 1024])
def test_kv_batch_d2d_small_pool(gpu, oracle, units):
    pool = 64 * MIB
    src, dst, lens = workloads.kv_batch(0xC1, pool)
    _check_d2d(gpu, oracle, pool, src, dst, lens, 0xC1, units)


@pytest.mark.parametrize("count,units", [(1, 0), (7, 256), (128, 0), (129, 0), (1000, 512), (5000, 0)])
def test_ragged_batches_d2d(gpu, oracle, count, units):
    """Arbitrary byte offsets and lengths (zeros included), below and above the 128-segment inline limit."""
    pool = 48 * MIB
    src, dst, lens = workloads.ragged_batch(count, pool, count, max_len=9000 if count > 200 else 70000)
    _check_d2d(gpu, oracle, pool, src, dst, lens, count, units)


def test_every_small_length_and_alignment_in_one_launch(gpu, oracle):
    """Lengths 0..257 x source alignment 0..15 x destination alignment {0,1,8,15}: 16 512 segments."""
    src_off, dst_off, lens = [], [], []
    s_cursor, d_cursor = 0, 0
    for length in range(258):
        for sa in range(16):
            for da in (0, 1, 8, 15):
                src_off.append(s_cursor + sa)
                dst_off.append(d_cursor + da)
                lens.append(length)
                s_cursor += 320
                d_cursor += 320
    half = (max(s_cursor, d_cursor) + 4095) // 4096 * 4096
    dst_off = [d + half for d in dst_off]
    _check_d2d(gpu, oracle, 2 * half, np.array(src_off), np.array(dst_off), np.array(lens), 0xA1)


@pytest.mark.parametrize("length,count", [(5000, 300), (32768, 700), (12288 + 7, 2000)])
def test_equal_sized_segments_at_ragged_places(gpu, oracle, length, count):
    """Segments of one size have equal chunk counts whatever their alignment: the launch that
    finds a chunk's segment by division instead of a search must move the same bytes."""
    rng = np.random.default_rng(length)
    slot = (length + 64 + 4095) // 4096 * 4096
    half = slot * count
    src_off = rng.permutation(count) * slot + rng.integers(0, 48, count)
    dst_off = half + np.arange(count) * slot + rng.integers(0, 48, count)
    _check_d2d(gpu, oracle, 2 * half, src_off, dst_off, np.full(count, length), length)


@pytest.mark.parametrize("sizes,count", [((131072, 16384), 610), ((5000, 70000, 12288), 999), ((4096,) * 7 + (40960,), 1203)])
def test_sizes_taking_turns_above_the_inline_limit(gpu, oracle, sizes, count):
    """K and V blocks in turn, several requests in one call: the chunk counts repeat with a short
    period, which the launch uses instead of a chunk prefix.  Placement is random, alignment ragged."""
    rng = np.random.default_rng(count)
    lens = np.array([sizes[i % len(sizes)] for i in range(count)])
    slot = (max(sizes) + 64 + 4095) // 4096 * 4096
    half = slot * count
    src_off = rng.permutation(count) * slot + rng.integers(0, 16, count) * (1 if min(sizes) % 4096 else 0)
    dst_off = half + rng.permutation(count) * slot + rng.integers(0, 16, count) * (1 if min(sizes) % 4096 else 0)
    _check_d2d(gpu, oracle, 2 * half, src_off, dst_off, lens, count)


def _held_case(rng, count, sizes, ragged):
    """count segments whose lengths take turns over `sizes` (+ a ragged few bytes), sources and destinations at
    random slots of the two halves of a pool; returns (pool bytes, src, dst, lens)."""
    lens = np.array([sizes[i % len(sizes)] for i in range(count)], dtype=np.uint64)
    if ragged:
        lens = lens - rng.integers(0, 3000, count).astype(np.uint64)
    slot = (int(lens.max()) + 64 + 4095) // 4096 * 4096
    half = slot * count
    odd = rng.integers(0, 16, count) if ragged else np.zeros(count, dtype=np.int64)
    src = rng.permutation(count) * slot + odd
    dst = half + rng.permutation(count) * slot + rng.integers(0, 16, count) * (1 if ragged else 0)
    return 2 * half, src, dst, lens


@pytest.mark.parametrize("count,sizes,ragged", [
    (244, (131072, 16384), False),      # 4392 chunks of 4 KiB out of a table: stores of four loads held
    (300, (65536, 20480), True),        # the same with a group map instead of a pattern
    (32, (1 << 20,), False),            # 32 MiB in the kernel arguments: 16 KiB per wave, stores of sixteen loads held
    (100, (400000,), True),             # the same with heads, tails and last chunks that are not whole
    (488, (131072, 16384), False),      # 36 MB out of a table under a pattern, 16 KiB per wave
    (400, (150000, 40000, 98304), True),  # 38 MB, ragged: group map, 16 KiB per wave
    (1, (16 << 20,), False),            # one segment of 16 MiB: 4096 chunks of 4 KiB, no table, stores of four loads held
    (1, ((9 << 20) + 777,), True),      # the same with a head, a tail and a last chunk that is not whole
    (1, (48 << 20,), False),            # one segment of 48 MiB
    (1, ((40 << 20) + 12345,), True),
    (976, (131072, 16384), False),      # 72 MB: beyond what the waves hold at once, the usual form
])
def test_batches_whose_stores_are_held_back(gpu, oracle, count, sizes, ragged):
    """Batches of 4 to 64 MiB between device addresses wait with their stores until the loads of the launch are out
    (4 KiB per wave up to 24 MiB, 16 KiB per wave beyond), whether their descriptors travel in the kernel
    arguments or in a table.  With the wait at its rule, forced absurdly long (so that every wave does
    wait) and off, the bytes are the oracle's."""
    rng = np.random.default_rng(count * 7 + len(sizes))
    pool, src, dst, lens = _held_case(rng, count, sizes, ragged)
    for hold in (-1, 9000, 0):
        assert gpu.mf_xcopy_hold_stores(hold) == 0
        try:
            _check_d2d(gpu, oracle, pool, src, dst, lens, count + hold + 1)
        finally:
            assert gpu.mf_xcopy_hold_stores(-1) == 0


@pytest.mark.parametrize("count", [16384, 70000])
def test_batches_at_and_beyond_the_reference_slot_size(gpu, oracle, count):
    """16 384 segments fill one parameter slot of the reference (hybm_data_op_sdma.cpp:25-31 there);
    this path takes any count in one call."""
    pool = 96 * MIB
    src, dst, lens = workloads.ragged_batch(count, pool, count, max_len=600)
    _check_d2d(gpu, oracle, pool, src, dst, lens, count)


def test_one_segment_longer_than_4gib(gpu, oracle):
    """A single copy whose length does not fit 32 bits (5 GiB + 5 bytes, odd offsets on both sides):
    the planner cuts it into pieces.  Source blocks differ from each other, so a piece that lands
    at a wrong offset cannot go unnoticed; the bytes around the destination must stay untouched."""
    n = 5 * (1 << 30) + 5
    block = _random_bytes(oracle, 64 * MIB, 0x5A1)
    blocks = (n + len(block) - 1) // len(block) + 1
    src = gpu_util.DeviceBuffer(gpu, blocks * len(block))
    dst = gpu_util.DeviceBuffer(gpu, n + 4096)
    try:
        for i in range(blocks):
            src.upload(block ^ np.uint8((i * 29 + 3) & 0xFF), i * len(block))
        dst.fill(0xEE)
        gpu_util.xcopy(gpu, np.array([src.ptr + 7], dtype=np.uint64), np.array([dst.ptr + 1001], dtype=np.uint64),
                       np.array([n], dtype=np.uint64), native.ROUTE_HBM)
        edge = dst.download(0, 1001)
        assert np.all(edge == 0xEE)
        edge = dst.download(1001 + n, 4096 - 1001)
        assert np.all(edge == 0xEE)
        step = 256 * MIB
        for at in range(0, n, step):
            take = min(step, n - at)
            got = dst.download(1001 + at, take)
            want = np.empty(take, dtype=np.uint8)
            pos = 0
            while pos < take:                      # rebuild the source bytes [7 + at + pos, ...) from the block pattern
                absolute = 7 + at + pos
                i, off = divmod(absolute, len(block))
                m = min(len(block) - off, take - pos)
                want[pos:pos + m] = block[off:off + m] ^ np.uint8((i * 29 + 3) & 0xFF)
                pos += m
            assert np.array_equal(got, want), at
    finally:
        src.free()
        dst.free()


def test_single_large_copy_with_odd_edges(gpu, oracle):
    pool = 192 * MIB
    _check_d2d(gpu, oracle, pool, np.array([3]), np.array([96 * MIB + 5]), np.array([80 * MIB + 123]), 0xB2)


def test_adjacent_segments_are_merged_without_changing_bytes(gpu, oracle):
    pool = 32 * MIB
    n = 300
    src = np.arange(n) * 4096 + 8192
    dst = np.arange(n) * 4096 + 16 * MIB
    lens = np.full(n, 4096)
    before = gpu.mf_xcopy_launch_count()
    _check_d2d(gpu, oracle, pool, src, dst, lens, 0xB3)
    assert gpu.mf_xcopy_launch_count() - before == 1  # one inline launch, not a 300-entry table


def test_pinned_host_routes(gpu, oracle):
    """H2D then D2H through mapped pinned memory, 122-segment KV shape."""
    pool = 64 * MIB
    host = gpu_util.PinnedBuffer(gpu, pool)
    back = gpu_util.PinnedBuffer(gpu, pool)
    dev = gpu_util.DeviceBuffer(gpu, pool)
    try:
        host.array[:] = _random_bytes(oracle, pool, 0xC1)
        back.array[:] = 0x11
        dev.fill(0x22)
        src, dst, lens = workloads.kv_batch(0xC1, pool, same_pool=False)
        gpu_util.xcopy(gpu, host.ptr + src, dev.ptr + dst, lens, native.ROUTE_FROM_HOST)
        got_dev = dev.download()
        expect_dev = np.full(pool, 0x22, dtype=np.uint8)
        gpu_util.oracle_batch(oracle, host.array, expect_dev, src, dst, lens)
        assert np.array_equal(got_dev, expect_dev)
        # and back out to a second pinned pool at the source offsets
        gpu_util.xcopy(gpu, dev.ptr + dst, back.ptr + src, lens, native.ROUTE_TO_HOST)
        expect_back = np.full(pool, 0x11, dtype=np.uint8)
        gpu_util.oracle_batch(oracle, expect_dev, expect_back, dst, src, lens)
        assert np.array_equal(back.array, expect_back)
    finally:
        dev.free()
        host.free()
        back.free()


def _device_table_case(kind, count, rng, pool):
    """(src, dst, lens) offsets of one table for the device-side planner."""
    half = pool // 2
    if kind == "ragged":
        return workloads.ragged_batch(count * 3 + 1, pool, count, max_len=min(9000, half // count - 64))
    slot = half // count // 64 * 64
    src = rng.permutation(count).astype(np.uint64) * np.uint64(slot)
    dst = np.uint64(half) + rng.permutation(count).astype(np.uint64) * np.uint64(slot)
    if kind == "pages":                       # one size: period 1
        lens = np.full(count, min(slot - 64, 20000), dtype=np.uint64)
    elif kind == "turns":                     # three sizes in turn, one of them empty: period 3 with an empty member
        sizes = (min(slot - 64, 9000), 0, min(slot - 64, 4096))
        lens = np.array([sizes[i % 3] for i in range(count)], dtype=np.uint64)
        src += rng.integers(0, 16, count).astype(np.uint64)
    elif kind == "gaps":                      # runs of empty segments longer than one probe round between live ones
        lens = np.zeros(count, dtype=np.uint64)
        live = rng.choice(count, size=max(2, count // 150), replace=False)
        lens[live] = rng.integers(1, slot - 64, len(live)).astype(np.uint64)
        dst += rng.integers(0, 16, count).astype(np.uint64)
    elif kind == "empty":
        lens = np.zeros(count, dtype=np.uint64)
    else:                                     # "long": one segment of many groups among short ones
        lens = rng.integers(0, min(slot - 64, 3000), count).astype(np.uint64)
        big = count // 2
        room = (count - big) * slot - 64
        lens[big] = min(room, 24 * MIB)
        lens[big + 1:] = 0
        src[big], dst[big] = big * slot, half + big * slot
        src[:big] = np.arange(big, dtype=np.uint64) * np.uint64(slot)
        dst[:big] = np.uint64(half) + np.arange(big, dtype=np.uint64) * np.uint64(slot)
    return src, dst, lens


@pytest.mark.parametrize("kind,count", [
    ("ragged", 3000), ("ragged", 1), ("ragged", 1000), ("ragged", 2048), ("ragged", 5000), ("ragged", 8192),
    ("ragged", 8193), ("ragged", 40000), ("pages", 700), ("pages", 9000), ("turns", 1500), ("turns", 20001),
    ("gaps", 6000), ("gaps", 30000), ("empty", 3000), ("long", 400), ("long", 12000),
])
def test_device_resident_table(gpu, oracle, kind, count):
    """A {src, dst, len} table the host cannot read is planned on the GPU: by one workgroup up to 8192 segments (1, 2, 4 or
    8 tiles of 1024), by one workgroup per 1024 segments beyond; chunk counts that repeat are found there and take the
    launch without a prefix, the rest the group map, whose groups empty segments and long segments stretch."""
    pool = 96 * MIB
    rng = np.random.default_rng(count + len(kind))
    src, dst, lens = _device_table_case(kind, count, rng, pool)
    init = _random_bytes(oracle, pool, count)
    buf = gpu_util.DeviceBuffer(gpu, pool)
    table = gpu_util.DeviceBuffer(gpu, count * 24)
    try:
        buf.upload(init)
        triples = np.empty((count, 3), dtype=np.uint64)
        triples[:, 0] = buf.ptr + src
        triples[:, 1] = buf.ptr + dst
        triples[:, 2] = lens
        table.upload(triples.view(np.uint8).reshape(-1))
        assert gpu.mf_xcopy_device_table(table.ptr, count, native.ROUTE_HBM, None) == 0, native.last_error()
        assert gpu.mfrt_device_sync() == 0
        got = buf.download()
    finally:
        buf.free()
        table.free()
    expect = init.copy()
    gpu_util.oracle_batch(oracle, init, expect, src, dst, lens)
    assert np.array_equal(got, expect)


def test_full_size_kv_batch_in_4gib_pool(gpu, oracle):
    """The benchmark's own shape: 4 GiB pool, 122 segments.  Touched ranges, their guard bands and
    64 MiB strides of the rest are compared; the pool is filled on the device side by copies of a
    256 MiB random block so that no 4 GiB host array is needed."""
    pool = 4 << 30
    block = 256 * MIB
    seed_block = _random_bytes(oracle, block, 0xC1)
    buf = gpu_util.DeviceBuffer(gpu, pool)
    try:
        for i in range(pool // block):
            buf.upload(seed_block, i * block)
        src, dst, lens = workloads.kv_batch(0xC1, pool)
        gpu_util.xcopy(gpu, buf.ptr + src, buf.ptr + dst, lens, native.ROUTE_HBM)
        guard = 4096
        for s, d, l in zip(src.tolist(), dst.tolist(), lens.tolist()):
            lo = max(0, d - guard)
            hi = min(pool, d + l + guard)
            got = buf.download(lo, hi - lo)
            expect = np.take(seed_block, np.arange(lo, hi) % block)
            expect[d - lo:d - lo + l] = np.take(seed_block, np.arange(s, s + l) % block)
            # neighbours of this destination may be other destinations: patch those too
            for s2, d2, l2 in zip(src.tolist(), dst.tolist(), lens.tolist()):
                a, b = max(lo, d2), min(hi, d2 + l2)
                if a < b:
                    expect[a - lo:b - lo] = np.take(seed_block, np.arange(s2 + a - d2, s2 + b - d2) % block)
            assert np.array_equal(got, expect), (s, d, l)
        for s, l in zip(src.tolist(), lens.tolist()):  # sources untouched
            assert np.array_equal(buf.download(s, l), np.take(seed_block, np.arange(s, s + l) % block))
    finally:
        buf.free()


def test_size_independent_properties_at_full_size(gpu, oracle):
    """Round trip and idempotence on the 1 GiB single copy: copy A->B, B->C, compare checksums of
    A and C computed from strided samples; copying again changes nothing."""
    n = 1 << 30
    a = gpu_util.DeviceBuffer(gpu, n)
    b = gpu_util.DeviceBuffer(gpu, n)
    try:
        block = _random_bytes(oracle, 64 * MIB, 0xC2)
        for i in range(n // len(block)):
            a.upload(block, i * len(block))
        b.fill(0)
        gpu_util.xcopy(gpu, [a.ptr], [b.ptr], [n], native.ROUTE_HBM)
        for off in range(0, n, 64 * MIB):
            assert np.array_equal(b.download(off, 64 * MIB), block)
        gpu_util.xcopy(gpu, [a.ptr], [b.ptr], [n], native.ROUTE_HBM)  # idempotent
        assert np.array_equal(b.download(n - 64 * MIB, 64 * MIB), block)
        # an odd-length, odd-offset slice inside the big buffers
        b.fill(0)
        gpu_util.xcopy(gpu, [a.ptr + 1], [b.ptr + 7], [n - 64], native.ROUTE_HBM)
        head = b.download(0, 4096)
        assert np.all(head[:7] == 0) and np.array_equal(head[7:], block[1:4090])
        tail = b.download(n - 4096, 4096)
        end = 7 + n - 64
        assert np.all(tail[end - (n - 4096):] == 0)
        assert np.array_equal(tail[:end - (n - 4096)], np.take(block, np.arange(n - 4096 - 6, n - 63) % len(block)))
    finally:
        a.free()
        b.free()
