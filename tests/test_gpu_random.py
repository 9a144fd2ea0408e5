"""Randomised cases on the GPU against plain numpy (copies) and the oracle (MoE): shapes, counts, alignments and
routings drawn from a seeded generator, so that no case owes its place to how the kernels are written.  The
hand-picked edge cases live in the other GPU test files; this one looks where nobody thought to."""

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu

POOL = 256 << 20


@pytest.fixture(scope="module")
def gpu(lib):
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    yield lib
    lib.hybm_uninit()


def _dev(gpu, array):
    a = np.ascontiguousarray(array)
    buf = gpu_util.DeviceBuffer(gpu, max(a.nbytes, 16))
    if a.nbytes:
        buf.upload(a.view(np.uint8).reshape(-1))
    return buf


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_batches_copy_exactly_their_bytes(gpu, seed):
    """Sixty batches per seed: a few long segments, up to 128 ragged ones, thousands of short ones, pages of one size,
    segments below 64 bytes, K and V blocks in turn; sources anywhere, destinations disjoint with gaps, alignment from
    1 to 4096 bytes, segments in shuffled order.  Every byte of the destination range is compared, the gaps included."""
    rng = np.random.default_rng(seed)
    src = gpu_util.DeviceBuffer(gpu, POOL)
    dst = gpu_util.DeviceBuffer(gpu, POOL)
    data = rng.integers(0, 256, POOL, dtype=np.uint8)
    src.upload(data)
    try:
        for it in range(60):
            kind = int(rng.integers(0, 6))
            if kind == 0:
                lens = rng.integers(0, 40 << 20, int(rng.integers(1, 8)))
            elif kind == 1:
                lens = rng.integers(0, 300000, int(rng.integers(1, 129)))
            elif kind == 2:
                lens = rng.integers(0, 60000, int(rng.integers(129, 3000)))
            elif kind == 3:
                lens = np.full(int(rng.integers(129, 2000)), int(rng.integers(1, 9)) * 4096)
            elif kind == 4:
                lens = rng.integers(0, 64, int(rng.integers(1, 300)))
            else:
                lens = np.where(rng.integers(0, 2, int(rng.integers(2, 400))) == 0, 131072, 16384)
            lens = lens.astype(np.int64)
            n = len(lens)
            if int(lens.sum()) + n * 8192 > POOL // 2:
                lens //= 4
            align = int(rng.choice([1, 1, 4, 16, 256, 4096]))
            gaps = rng.integers(0, 4096, n)
            d_off = np.zeros(n, dtype=np.int64)
            pos = int(rng.integers(0, 4096))
            for i in range(n):
                pos = (pos + int(gaps[i]) + align - 1) // align * align
                d_off[i] = pos
                pos += int(lens[i])
            assert pos <= POOL
            s_off = np.array([int(rng.integers(0, POOL - int(l) - 4096)) // align * align + (int(rng.integers(0, 16)) if align == 1 else 0)
                              for l in lens], dtype=np.int64)
            perm = rng.permutation(n)
            dst.fill(0xA5)
            ret = gpu.mf_xcopy_batch(native.u64_array((src.ptr + s_off[perm]).tolist()), native.u64_array((dst.ptr + d_off[perm]).tolist()),
                                     native.u64_array(lens[perm].tolist()), n, native.ROUTE_HBM, None)
            assert ret == 0, native.last_error()
            assert gpu.mfrt_device_sync() == 0
            expect = np.full(pos, 0xA5, dtype=np.uint8)
            for i in range(n):
                expect[d_off[i]:d_off[i] + lens[i]] = data[s_off[i]:s_off[i] + lens[i]]
            assert np.array_equal(dst.download(0, pos), expect), (seed, it, kind, n, align)
    finally:
        src.free()
        dst.free()


@pytest.mark.parametrize("seed", [21, 22])
def test_random_moe_shapes_against_the_oracle(gpu, oracle, seed):
    """Twenty-five shapes per seed: fan-in 1 to 16, 1 to 512 experts, rows of 8 to 16 384 elements (whole cache lines
    and not), 1 to 20 000 tokens, a third of the cases with expert ids out of range.  Dispatch: row map, counts and
    every routed row bit-exact, rows nobody was sent to untouched.  Combine: on rows that differ within a token, with
    the GPU's own row map, bit-equal to the oracle."""
    rng = np.random.default_rng(seed)
    for it in range(25):
        K = int(rng.choice([1, 2, 3, 4, 6, 8, 8, 8, 16]))
        E = int(rng.choice([1, 2, 8, 37, 64, 128, 256, 300, 512]))
        H = int(rng.choice([8, 64, 520, 1024, 1600, 2048, 4096, 5120, 7168, 8192, 8256, 10000, 12288, 16384]))
        T = int(rng.integers(1, max(1, min(20000, (160 << 20) // (K * H * 2))) + 1))
        case = (seed, it, T, H, K, E)
        x = workloads.f32_to_bf16_words(rng.standard_normal((T, H), dtype=np.float32))
        topk = rng.integers(0, E, (T, K)).astype(np.int32)
        if rng.integers(0, 3) == 0:
            nbad = int(rng.integers(1, 50))
            topk[rng.integers(0, T, nbad), rng.integers(0, K, nbad)] = rng.choice([-1, E, E + 7])
        invalid = (topk < 0) | (topk >= E)
        # the oracle refuses ids out of range: it gets them as one more expert behind the real ones
        fixed = np.ascontiguousarray(np.where(invalid, E, topk).astype(np.int32))
        out = np.zeros((T * K, H), dtype=np.uint16)
        counts = np.zeros(E + 1, dtype=np.int32)
        offsets = np.zeros(E + 1, dtype=np.int32)
        row_of = np.zeros(T * K, dtype=np.int32)
        src_of = np.zeros(T * K, dtype=np.int32)
        assert oracle.orc_moe_dispatch(np_ptr(x), np_ptr(fixed), T, H, K, E + 1, np_ptr(out), np_ptr(counts), np_ptr(offsets),
                                       np_ptr(row_of), np_ptr(src_of)) == 0
        exp_row = np.ascontiguousarray(np.where(invalid.reshape(-1), -1, row_of).astype(np.int32))
        valid = int(counts[:E].sum())
        ws_bytes = gpu.mf_moe_workspace_bytes(T, K, E)
        bufs = [_dev(gpu, x), _dev(gpu, topk), gpu_util.DeviceBuffer(gpu, max(T * K * H * 2, 16)), gpu_util.DeviceBuffer(gpu, E * 4),
                gpu_util.DeviceBuffer(gpu, E * 4), gpu_util.DeviceBuffer(gpu, T * K * 4), gpu_util.DeviceBuffer(gpu, T * K * 4),
                gpu_util.DeviceBuffer(gpu, ws_bytes)]
        dx, dt, dout, dcounts, doffsets, drow, dsrc, dws = bufs
        dws.fill(0xFF)
        dout.fill(0x77)
        try:
            assert gpu.mf_moe_dispatch(dx.ptr, dt.ptr, T, H, K, E, dout.ptr, dcounts.ptr, doffsets.ptr, drow.ptr, dsrc.ptr, dws.ptr,
                                       ws_bytes, None) == 0, native.last_error()
            assert gpu.mfrt_device_sync() == 0
            assert np.array_equal(drow.download(0, T * K * 4).view(np.int32), exp_row), case
            assert np.array_equal(dcounts.download(0, E * 4).view(np.int32), counts[:E]), case
            assert dws.download(0, 4).view(np.uint32)[0] == (1 if invalid.any() else 0), case
            got = dout.download(0, T * K * H * 2).view(np.uint16).reshape(T * K, H)
            assert np.array_equal(got[:valid], out[:valid]), case
            assert np.all(got[valid:] == 0x7777), case
            del got
            w = rng.random((T, K), dtype=np.float32)
            rows = (rng.integers(0x3800, 0x4000, (T * K, H), dtype=np.uint16) | (rng.integers(0, 2, (T * K, H), dtype=np.uint16) << 15))
            exp_y = np.zeros((T, H), dtype=np.uint16)
            oracle.orc_moe_combine(np_ptr(rows), np_ptr(exp_row), np_ptr(w), T, H, K, np_ptr(exp_y))
            drows, dw, dy = _dev(gpu, rows), _dev(gpu, w), gpu_util.DeviceBuffer(gpu, T * H * 2)
            bufs += [drows, dw, dy]
            assert gpu.mf_moe_combine(drows.ptr, drow.ptr, dw.ptr, T, H, K, dy.ptr, None) == 0, native.last_error()
            assert gpu.mfrt_device_sync() == 0
            assert np.array_equal(dy.download(0, T * H * 2).view(np.uint16).reshape(T, H), exp_y), case
        finally:
            for b in bufs:
                b.free()


@pytest.mark.parametrize("seed", [31, 32])
def test_random_rectangles_side_by_side_and_alone(gpu, seed):
    """Twenty batches per seed of 1 to 200 rectangles: groups of two or three column blocks laid side by side in the
    destination (the first two of a group of one shape share their chunks in turn inside the kernel; a third, or one
    of another height, does not), blocks alone, widths from one unit to rows wider than a chunk, some unaligned
    (those go row by row).  Every destination byte is compared, the space between rectangles included."""
    rng = np.random.default_rng(seed)
    src_bytes, dst_bytes = 32 << 20, 96 << 20
    data = rng.integers(0, 256, src_bytes, dtype=np.uint8)
    sbuf = gpu_util.DeviceBuffer(gpu, src_bytes)
    dbuf = gpu_util.DeviceBuffer(gpu, dst_bytes)
    sbuf.upload(data)
    try:
        for it in range(20):
            rects, model = [], []
            cursor = int(rng.integers(0, 64)) * 16
            groups = int(rng.integers(1, 80))
            for _ in range(groups):
                blocks = int(rng.choice([1, 1, 2, 2, 2, 3]))
                width = int(rng.choice([16, 48, 896, 1000, 2368, 4736, 20000, 40000]))
                if rng.integers(0, 8) == 0:
                    width += int(rng.integers(1, 16))           # unaligned: row by row
                height = int(rng.integers(1, 120))
                dpitch = blocks * width + int(rng.integers(0, 3)) * 16
                used = 0
                for b in range(blocks):
                    h = height if b < 2 or rng.integers(0, 2) == 0 else max(1, height - int(rng.integers(1, 5)))
                    spitch = width + int(rng.integers(0, 4)) * 16
                    soff = int(rng.integers(0, src_bytes - spitch * h - 64)) // 16 * 16
                    if width % 16 != 0:
                        soff += int(rng.integers(0, 16))
                    rects.append((sbuf.ptr + soff, dbuf.ptr + cursor + b * width, width, h, spitch, dpitch))
                    model.append((soff, cursor + b * width, width, h, spitch, dpitch))
                    used = max(used, dpitch * h)
                cursor += (used + 255) // 256 * 256
                if cursor > dst_bytes - (8 << 20):
                    break
            descs = (native.Copy2dDesc * len(rects))()
            for i, r in enumerate(rects):
                descs[i] = native.Copy2dDesc(*[int(v) for v in r])
            dbuf.fill(0x3D)
            assert gpu.mf_xcopy_2d_batch(descs, len(rects), native.ROUTE_HBM, None) == 0, native.last_error()
            assert gpu.mfrt_device_sync() == 0
            expect = np.full(cursor, 0x3D, dtype=np.uint8)
            for soff, doff, width, h, spitch, dpitch in model:
                rows_src = np.lib.stride_tricks.as_strided(data[soff:], shape=(h, width), strides=(spitch, 1))
                rows_dst = np.lib.stride_tricks.as_strided(expect[doff:], shape=(h, width), strides=(dpitch, 1))
                rows_dst[:] = rows_src
            assert np.array_equal(dbuf.download(0, cursor), expect), (seed, it, len(rects))
    finally:
        sbuf.free()
        dbuf.free()
