"""GPU parity of the local MoE dispatch / combine against the CPU specification in
oracle/mf_oracle.c.  Dispatch is integer/byte work: bit-exact.  Combine is floating point: the
stated tolerance is 1e-2 relative (bf16); because both sides use the same fp32 FMA chain and one
final rounding, the test additionally demands bit-equality, which is the stronger statement."""

import ctypes

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu


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


def _fetch(buf, dtype, shape):
    n = int(np.prod(shape)) * np.dtype(dtype).itemsize
    return buf.download(0, n).view(dtype).reshape(shape)


def _oracle_dispatch(oracle, x, topk, E):
    T, H = x.shape
    K = topk.shape[1]
    out = np.zeros((T * K, H), dtype=np.uint16)
    counts = np.zeros(E, dtype=np.int32)
    offsets = np.zeros(E, dtype=np.int32)
    row_of = np.zeros(T * K, dtype=np.int32)
    src_of = np.zeros(T * K, dtype=np.int32)
    ret = oracle.orc_moe_dispatch(np_ptr(x), np_ptr(topk), T, H, K, E, np_ptr(out), np_ptr(counts), np_ptr(offsets),
                                  np_ptr(row_of), np_ptr(src_of))
    assert ret == 0
    return out, counts, offsets, row_of, src_of


def _gpu_dispatch(gpu, x, topk, E, with_rows=True):
    T, H = x.shape
    K = topk.shape[1]
    ws_bytes = gpu.mf_moe_workspace_bytes(T, K, E)
    bufs = {
        "x": _dev(gpu, x), "topk": _dev(gpu, topk), "out": gpu_util.DeviceBuffer(gpu, max(T * K * H * 2, 16)),
        "counts": gpu_util.DeviceBuffer(gpu, E * 4), "offsets": gpu_util.DeviceBuffer(gpu, E * 4),
        "row_of": gpu_util.DeviceBuffer(gpu, T * K * 4), "src_of": gpu_util.DeviceBuffer(gpu, T * K * 4),
        "ws": gpu_util.DeviceBuffer(gpu, ws_bytes),
    }
    bufs["ws"].fill(0xFF)  # the workspace needs no initialisation
    bufs["src_of"].fill(0xFF)
    ret = gpu.mf_moe_dispatch(bufs["x"].ptr if with_rows else None, bufs["topk"].ptr, T, H, K, E,
                              bufs["out"].ptr if with_rows else None, bufs["counts"].ptr, bufs["offsets"].ptr,
                              bufs["row_of"].ptr, bufs["src_of"].ptr, bufs["ws"].ptr, ws_bytes, None)
    assert ret == 0, native.last_error()
    assert gpu.mfrt_device_sync() == 0
    return bufs


def _free(bufs):
    for b in bufs.values():
        b.free()


def _inputs(oracle, seed, T, H, K, E):
    x, logits = workloads.moe_inputs(seed, T, H, E, K)
    topk = np.zeros((T, K), dtype=np.int32)
    w = np.zeros((T, K), dtype=np.float32)
    oracle.orc_moe_route(np_ptr(logits), T, E, K, np_ptr(topk), np_ptr(w))
    return x, topk, w


@pytest.mark.parametrize("T,H,K,E", [
    (1, 8, 1, 1), (7, 64, 2, 4), (300, 64, 4, 16), (1000, 520, 8, 256), (129, 1024, 8, 300),
    (2050, 72, 16, 512), (4096, 2048, 8, 256), (511, 16384, 3, 37),
    (40000, 64, 8, 300),   # 320 000 entries in 313 rank blocks
    (5000, 8192, 2, 8),    # wide rows in two parts: every wave of the permute takes two or three (token, part) items
])
def test_dispatch_and_combine_match_the_specification(gpu, oracle, T, H, K, E):
    K = min(K, E)
    x, topk, w = _inputs(oracle, 0xC4 + T, T, H, K, E)
    exp_out, exp_counts, exp_offsets, exp_row, exp_src = _oracle_dispatch(oracle, x, topk, E)
    bufs = _gpu_dispatch(gpu, x, topk, E)
    try:
        assert np.array_equal(_fetch(bufs["counts"], np.int32, (E,)), exp_counts)
        assert np.array_equal(_fetch(bufs["offsets"], np.int32, (E,)), exp_offsets)
        assert np.array_equal(_fetch(bufs["row_of"], np.int32, (T * K,)), exp_row)
        assert np.array_equal(_fetch(bufs["src_of"], np.int32, (T * K,)), exp_src)
        assert np.array_equal(_fetch(bufs["out"], np.uint16, (T * K, H)), exp_out)
        assert _fetch(bufs["ws"], np.uint32, (1,))[0] == 0

        wdev = _dev(gpu, w)
        y = gpu_util.DeviceBuffer(gpu, T * H * 2)
        assert gpu.mf_moe_combine(bufs["out"].ptr, bufs["row_of"].ptr, wdev.ptr, T, H, K, y.ptr, None) == 0
        assert gpu.mfrt_device_sync() == 0
        got = _fetch(y, np.uint16, (T, H))
        exp_y = np.zeros((T, H), dtype=np.uint16)
        oracle.orc_moe_combine(np_ptr(exp_out), np_ptr(exp_row), np_ptr(w), T, H, K, np_ptr(exp_y))
        gf = workloads.bf16_words_to_f32(got).astype(np.float64)
        ef = workloads.bf16_words_to_f32(exp_y).astype(np.float64)
        assert np.all(np.abs(gf - ef) <= 1e-2 * np.abs(ef) + 1e-6)   # the stated tolerance
        assert np.array_equal(got, exp_y)                             # and in fact bit-equal
        wdev.free()
        y.free()
    finally:
        _free(bufs)


@pytest.mark.parametrize("T,H,K,E,routing", [
    (2000, 4096, 8, 64, "router"),     # 16 000 entries: fifteen full blocks and a last one of 640 entries
    (2500, 7168, 8, 300, "router"),    # twenty blocks, which the eight streams do not divide
    (2200, 7168, 8, 256, "five"),      # everything lands on five experts, duplicates inside a token included: long runs
    (2200, 5120, 8, 256, "bad ids"),   # some ids out of range: their slots name no row, the lists of their blocks are shorter
    (1200, 4096, 16, 128, "router"),   # sixty-four tokens per block
    (2800, 4096, 6, 64, "router"),     # blocks that begin and end inside a token
    (3000, 8256, 8, 1, "one"),         # one expert: the output is the input, every row eight times; rows that end inside a tile
    (2100, 16384, 8, 256, "router"),   # rows so wide that a step is half a block of entries
    (6000, 4096, 2, 8, "router"),      # top-2: 512 tokens per block, steps of half a block
    (2500, 12288, 8, 512, "bad ids"),  # 512 experts, half-block steps, slots without a row
    (700, 16384, 3, 37, "router"),     # steps of two slices (128 entries) that begin and end inside tokens
    (2100, 1024, 8, 32, "router"),     # rows of one tile
    (4000, 1600, 5, 100, "bad ids"),   # rows of one tile and a part of one
])
def test_output_ordered_permute(gpu, oracle, T, H, K, E, routing):
    """Rows wide enough and blocks enough for the permute that walks the output in runs of consecutive rows per
    expert, in tiles: every output row and every map against the oracle."""
    assert gpu.mf_moe_xcd_streams() == 1        # an MI355X in its default partition: the form under test is the one that runs
    x, topk, _ = _inputs(oracle, 0xD1 + T, T, H, min(K, E), E)
    rng = np.random.default_rng(T)
    if routing == "one":
        topk = np.zeros((T, K), dtype=np.int32)
    elif routing == "five":
        topk = rng.integers(0, 5, (T, K)).astype(np.int32)
        topk[::7, 0] = E - 1
    elif routing == "bad ids":
        topk = topk.copy()
        topk[rng.integers(0, T, 300), rng.integers(0, K, 300)] = E + 3
        topk[5, :] = -1                                     # a token nobody takes
    if routing == "bad ids":
        # the oracle refuses ids out of range; it is asked about the same routing with those entries sent to one
        # more expert behind the others, which leaves every row of the real experts where it is
        bad = (topk < 0) | (topk >= E)
        exp_out, exp_counts, exp_offsets, exp_row, exp_src = _oracle_dispatch(oracle, x, np.where(bad, E, topk).astype(np.int32), E + 1)
        exp_counts, exp_offsets = exp_counts[:E], exp_offsets[:E]
        exp_row = np.where(bad.reshape(-1), -1, exp_row)
    else:
        exp_out, exp_counts, exp_offsets, exp_row, exp_src = _oracle_dispatch(oracle, x, topk, E)
    bufs = _gpu_dispatch(gpu, x, topk, E)
    try:
        valid = int(exp_counts.sum())
        assert np.array_equal(_fetch(bufs["counts"], np.int32, (E,)), exp_counts)
        assert np.array_equal(_fetch(bufs["offsets"], np.int32, (E,)), exp_offsets)
        assert np.array_equal(_fetch(bufs["row_of"], np.int32, (T * K,)), exp_row)
        assert np.array_equal(_fetch(bufs["src_of"], np.int32, (T * K,))[:valid], exp_src[:valid])
        assert np.array_equal(_fetch(bufs["out"], np.uint16, (T * K, H))[:valid], exp_out[:valid])
        assert _fetch(bufs["ws"], np.uint32, (1,))[0] == (1 if routing == "bad ids" else 0)
    finally:
        _free(bufs)


def test_skewed_routing_with_empty_and_hot_experts(gpu, oracle):
    rng = np.random.default_rng(3)
    T, H, K, E = 3000, 128, 8, 256
    x, _ = workloads.moe_inputs(3, T, H, E, K)
    topk = rng.integers(0, 5, (T, K)).astype(np.int32)       # everything lands on 5 experts, duplicates included
    topk[::7, 0] = 255
    exp_out, exp_counts, exp_offsets, exp_row, exp_src = _oracle_dispatch(oracle, x, topk, E)
    bufs = _gpu_dispatch(gpu, x, topk, E)
    try:
        assert np.array_equal(_fetch(bufs["counts"], np.int32, (E,)), exp_counts)
        assert np.array_equal(_fetch(bufs["row_of"], np.int32, (T * K,)), exp_row)
        assert np.array_equal(_fetch(bufs["out"], np.uint16, (T * K, H)), exp_out)
    finally:
        _free(bufs)


@pytest.mark.parametrize("T,K,E", [(300, 8, 256), (600, 8, 64), (1024, 8, 512), (2048, 2, 8), (1100, 5, 17), (1025, 8, 256)])
def test_few_blocks_that_count_one_anothers_entries(gpu, oracle, T, K, E):
    """Two to eight blocks of 1024 entries rank without a histogram launch: each block counts the entries of the
    others.  Everything against the oracle, then with one id out of range in the last block only (block 0 has to
    find it for the status word), then clean again."""
    H = 1024
    x, topk, _ = _inputs(oracle, 0xF0 + T, T, H, K, E)
    exp_out, exp_counts, exp_offsets, exp_row, exp_src = _oracle_dispatch(oracle, x, topk, E)
    bufs = _gpu_dispatch(gpu, x, topk, E)
    try:
        assert _fetch(bufs["ws"], np.uint32, (1,))[0] == 0
        assert np.array_equal(_fetch(bufs["counts"], np.int32, (E,)), exp_counts)
        assert np.array_equal(_fetch(bufs["offsets"], np.int32, (E,)), exp_offsets)
        assert np.array_equal(_fetch(bufs["row_of"], np.int32, (T * K,)), exp_row)
        assert np.array_equal(_fetch(bufs["src_of"], np.int32, (T * K,)), exp_src)
        assert np.array_equal(_fetch(bufs["out"], np.uint16, (T * K, H)), exp_out)
    finally:
        _free(bufs)
    late = topk.copy()
    late[T - 1, K - 1] = E + 7
    sent = np.where(late >= E, E, late).astype(np.int32)
    exp_out, exp_counts, _, exp_row, _ = _oracle_dispatch(oracle, x, sent, E + 1)
    exp_row = np.where((late >= E).reshape(-1), -1, exp_row)
    bufs = _gpu_dispatch(gpu, x, late, E)
    try:
        assert _fetch(bufs["ws"], np.uint32, (1,))[0] == 1
        assert np.array_equal(_fetch(bufs["counts"], np.int32, (E,)), exp_counts[:E])
        assert np.array_equal(_fetch(bufs["row_of"], np.int32, (T * K,)), exp_row)
        assert np.array_equal(_fetch(bufs["out"], np.uint16, (T * K - 1, H)), exp_out[:T * K - 1])
    finally:
        _free(bufs)
    bufs = _gpu_dispatch(gpu, x, topk, E)
    try:
        assert _fetch(bufs["ws"], np.uint32, (1,))[0] == 0
    finally:
        _free(bufs)


def test_out_of_range_expert_ids_are_flagged_not_followed(gpu, oracle):
    T, H, K, E = 500, 64, 4, 32
    x, topk, _ = _inputs(oracle, 9, T, H, K, E)
    bad = topk.copy()
    bad[10, 1] = E
    bad[499, 3] = -3
    bufs = _gpu_dispatch(gpu, x, bad, E)
    try:
        assert _fetch(bufs["ws"], np.uint32, (1,))[0] == 1
        row_of = _fetch(bufs["row_of"], np.int32, (T * K,))
        assert row_of[10 * K + 1] == -1 and row_of[499 * K + 3] == -1
        good = np.delete(np.arange(T * K), [10 * K + 1, 499 * K + 3])
        assert sorted(row_of[good].tolist()) == list(range(T * K - 2))
        assert _fetch(bufs["counts"], np.int32, (E,)).sum() == T * K - 2
        # combine skips the two slots: with a NaN and an infinity in row 0 of the expert-contiguous
        # buffer the result still equals the oracle's, and nothing non-finite appears in y
        rows = _fetch(bufs["out"], np.uint16, (T * K, H)).copy()
        rows[T * K - 2:] = 0        # the two rows nobody was sent to
        row_of = row_of.copy()
        victim = int(np.where(row_of == 0)[0][0])
        rows[0, 0::2] = 0x7FC0
        rows[0, 1::2] = 0x7F80
        row_of[victim] = 1          # nobody reads the poisoned row
        w = np.random.default_rng(10).random((T, K), dtype=np.float32)
        rdev, rodev, wdev = _dev(gpu, rows), _dev(gpu, row_of), _dev(gpu, w)
        y = gpu_util.DeviceBuffer(gpu, T * H * 2)
        assert gpu.mf_moe_combine(rdev.ptr, rodev.ptr, wdev.ptr, T, H, K, y.ptr, None) == 0
        assert gpu.mfrt_device_sync() == 0
        got = _fetch(y, np.uint16, (T, H))
        exp_y = np.zeros((T, H), dtype=np.uint16)
        oracle.orc_moe_combine(np_ptr(rows), np_ptr(row_of), np_ptr(w), T, H, K, np_ptr(exp_y))
        assert np.array_equal(got, exp_y)
        assert not np.any((got & 0x7F80) == 0x7F80)
        for b in (rdev, rodev, wdev, y):
            b.free()
    finally:
        _free(bufs)
    # the same call with valid ids clears the flag again without any reset by the caller
    bufs = _gpu_dispatch(gpu, x, topk, E)
    try:
        assert _fetch(bufs["ws"], np.uint32, (1,))[0] == 0
    finally:
        _free(bufs)


@pytest.mark.parametrize("T,H,K", [
    (3600, 7168, 8),   # 25 200 slices: one full period for 4096 waves and a last period of two read parts and a short third
    (3300, 8000, 8),   # rows of 1000 units in eight slices of 125: ragged slices, a last period of three read parts
    (700, 1024, 8),    # narrow rows: one four-wave workgroup per token
    (60, 7168, 8),     # wide rows, few tokens: one workgroup per slice
    (300, 16384, 3),   # any other topK
    (500, 4096, 2),    # the slice kernel compiled for top-2
    (400, 7168, 4),    # ... top-4
    (300, 5120, 6),    # ... top-6
    (5100, 5120, 6),   # top-6, 25 500 slices: waves that stay, as in the first shape
    (3600, 7168, 4),   # top-4 with as many slices: still one workgroup per slice
])
def test_combine_of_rows_that_differ_within_a_token(gpu, oracle, T, H, K):
    """After a dispatch the rows of a token are copies of one another, so a combine that mixed them up would still pass
    the dispatch-then-combine tests; here every row is different.  The first two shapes and the top-6 shape of 5100 tokens have enough tokens of wide rows
    for the combine whose waves stay and alternate between reading and writing: same bits as the oracle at the
    default pace, at a slow and at an absurdly fast one, with slots without a row, and with the form switched off."""
    rng = np.random.default_rng(T)
    rows = (rng.integers(0x3800, 0x4000, (T * K, H), dtype=np.uint16) | (rng.integers(0, 2, (T * K, H), dtype=np.uint16) << 15))
    row_of = rng.permutation(T * K).astype(np.int32)
    row_of[rng.integers(0, T * K, 50)] = -1
    victim = int(np.where(row_of == 0)[0][0]) if np.any(row_of == 0) else None
    if victim is not None:
        row_of[victim] = 1                      # nobody reads row 0, which holds a NaN and an infinity
    rows[0, 0::2] = 0x7FC0
    rows[0, 1::2] = 0x7F80
    w = rng.random((T, K), dtype=np.float32)
    exp_y = np.zeros((T, H), dtype=np.uint16)
    oracle.orc_moe_combine(np_ptr(rows), np_ptr(row_of), np_ptr(w), T, H, K, np_ptr(exp_y))
    rdev, rodev, wdev = _dev(gpu, rows), _dev(gpu, row_of), _dev(gpu, w)
    y = gpu_util.DeviceBuffer(gpu, T * H * 2)
    try:
        for rates in (native.MOE_COMBINE_WINDOWS_DEFAULT, (1000000, 1000000), (16000000, 16000000), (0, 0)):
            assert gpu.mf_moe_combine_windows(*rates) == 0, native.last_error()
            y.fill(0xEE)
            assert gpu.mf_moe_combine(rdev.ptr, rodev.ptr, wdev.ptr, T, H, K, y.ptr, None) == 0, native.last_error()
            assert gpu.mfrt_device_sync() == 0
            got = _fetch(y, np.uint16, (T, H))
            assert np.array_equal(got, exp_y), rates
            assert not np.any((got & 0x7F80) == 0x7F80)
        assert gpu.mf_moe_combine_windows(500, 6500000) == native.BM_INVALID_PARAM
        assert gpu.mf_moe_combine_windows(0, 6500000) == native.BM_INVALID_PARAM
    finally:
        assert gpu.mf_moe_combine_windows(*native.MOE_COMBINE_WINDOWS_DEFAULT) == 0
        for b in (rdev, rodev, wdev, y):
            b.free()


def test_same_workspace_reused_by_calls_of_different_sizes(gpu, oracle):
    """Histograms and status of one call must not leak into the next call on the same workspace."""
    E, K, H = 64, 4, 64
    sizes = [5000, 700, 5000, 33]
    ws_bytes = gpu.mf_moe_workspace_bytes(max(sizes), K, E)
    ws = gpu_util.DeviceBuffer(gpu, ws_bytes)
    ws.fill(0xFF)
    try:
        for i, T in enumerate(sizes):
            x, topk, _ = _inputs(oracle, 0xB0 + i, T, H, K, E)
            _, exp_counts, exp_offsets, exp_row, _ = _oracle_dispatch(oracle, x, topk, E)
            dt = _dev(gpu, topk)
            counts, offsets = gpu_util.DeviceBuffer(gpu, E * 4), gpu_util.DeviceBuffer(gpu, E * 4)
            row_of = gpu_util.DeviceBuffer(gpu, T * K * 4)
            assert gpu.mf_moe_dispatch(None, dt.ptr, T, H, K, E, None, counts.ptr, offsets.ptr, row_of.ptr, None, ws.ptr,
                                       ws_bytes, None) == 0, native.last_error()
            assert gpu.mfrt_device_sync() == 0
            assert np.array_equal(_fetch(counts, np.int32, (E,)), exp_counts)
            assert np.array_equal(_fetch(offsets, np.int32, (E,)), exp_offsets)
            assert np.array_equal(_fetch(row_of, np.int32, (T * K,)), exp_row)
            for b in (dt, counts, offsets, row_of):
                b.free()
    finally:
        ws.free()


def test_argument_errors(gpu):
    p = ctypes.c_void_p(0x1000)
    assert gpu.mf_moe_dispatch(p, None, 4, 8, 2, 4, p, p, p, p, None, p, 1 << 20, None) == native.BM_INVALID_PARAM
    assert gpu.mf_moe_dispatch(p, p, 4, 12, 2, 4, p, p, p, p, None, p, 1 << 20, None) == native.BM_INVALID_PARAM
    assert gpu.mf_moe_dispatch(p, p, 4, 8, 17, 4, p, p, p, p, None, p, 1 << 20, None) == native.BM_INVALID_PARAM
    assert gpu.mf_moe_dispatch(p, p, 4, 8, 2, 513, p, p, p, p, None, p, 1 << 20, None) == native.BM_INVALID_PARAM
    assert gpu.mf_moe_dispatch(p, p, 4, 8, 2, 4, p, p, p, p, None, p, 8, None) == native.BM_INVALID_PARAM
    assert gpu.mf_moe_combine(p, p, None, 4, 8, 2, p, None) == native.BM_INVALID_PARAM
    assert gpu.mf_moe_combine(p, p, p, 4, 9, 2, p, None) == native.BM_INVALID_PARAM


def test_full_size_local_share(gpu, oracle):
    """8192 tokens x 7168 bf16, 256 experts, top-8: whole outputs against the oracle, plus the
    size-independent properties (bijection, counts, one-hot combine returns the token)."""
    T, H, K, E = 8192, 7168, 8, 256
    x, topk, w = _inputs(oracle, 0xC4, T, H, K, E)
    exp_out, exp_counts, exp_offsets, exp_row, exp_src = _oracle_dispatch(oracle, x, topk, E)
    bufs = _gpu_dispatch(gpu, x, topk, E)
    try:
        row_of = _fetch(bufs["row_of"], np.int32, (T * K,))
        counts = _fetch(bufs["counts"], np.int32, (E,))
        assert counts.sum() == T * K
        assert np.array_equal(np.sort(row_of), np.arange(T * K))
        assert np.array_equal(counts, exp_counts)
        assert np.array_equal(_fetch(bufs["offsets"], np.int32, (E,)), exp_offsets)
        assert np.array_equal(row_of, exp_row)
        assert np.array_equal(_fetch(bufs["src_of"], np.int32, (T * K,)), exp_src)
        got_out = _fetch(bufs["out"], np.uint16, (T * K, H))
        assert np.array_equal(got_out, exp_out)
        del got_out

        wdev = _dev(gpu, w)
        y = gpu_util.DeviceBuffer(gpu, T * H * 2)
        assert gpu.mf_moe_combine(bufs["out"].ptr, bufs["row_of"].ptr, wdev.ptr, T, H, K, y.ptr, None) == 0
        assert gpu.mfrt_device_sync() == 0
        got = _fetch(y, np.uint16, (T, H))
        exp_y = np.zeros((T, H), dtype=np.uint16)
        oracle.orc_moe_combine(np_ptr(exp_out), np_ptr(exp_row), np_ptr(w), T, H, K, np_ptr(exp_y))
        gf = workloads.bf16_words_to_f32(got)
        ef = workloads.bf16_words_to_f32(exp_y)
        assert np.all(np.abs(gf - ef) <= 1e-2 * np.abs(ef) + 1e-6)
        assert np.array_equal(got, exp_y)
        # one-hot weights: combine(dispatch(x)) == x
        onehot = np.zeros((T, K), dtype=np.float32)
        onehot[:, 5] = 1.0
        wdev.upload(onehot.view(np.uint8).reshape(-1))
        assert gpu.mf_moe_combine(bufs["out"].ptr, bufs["row_of"].ptr, wdev.ptr, T, H, K, y.ptr, None) == 0
        assert gpu.mfrt_device_sync() == 0
        back = _fetch(y, np.uint16, (T, H))
        # the chain starts from +0, so a -0.0 input comes back as +0.0 (as it does in the oracle)
        assert np.array_equal(np.where(back == 0x8000, 0, back), np.where(x == 0x8000, 0, x))
        wdev.free()
        y.free()
    finally:
        _free(bufs)
