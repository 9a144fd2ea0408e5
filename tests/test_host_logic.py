"""Host-side logic of the product (no GPU): direction algebra, window arithmetic,
work decomposition and the error contracts of the C API, each against the oracle."""

import ctypes

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from tests.oracle_lib import np_ptr, ptr_array, u64_array


# ---- direction algebra vs the reference's literal tables -----------------------------
def test_compose_direction_equals_infer_table(lib, oracle):
    cat = {0: (1, 1), 1: (1, 0), 2: (0, 1), 3: (0, 0)}  # category -> (pool, device)
    for s in range(4):
        for d in range(4):
            assert lib.mf_dir_compose(*cat[s], *cat[d]) == oracle.orc_infer_table(s, d)


def test_translate_smem_equals_direct_map_for_every_copy_type(lib, oracle):
    for copy_type in range(10):
        for s in range(5):
            for d in range(5):
                assert lib.mf_dir_translate_smem(copy_type, s, d) == oracle.orc_trans_direction(copy_type, s, d), \
                    (copy_type, s, d)


def test_direction_checks_equal_check_map(lib, oracle):
    for direction in range(14):
        got = lib.mf_dir_checks(direction)
        assert (got & 1) == oracle.orc_check_map(direction, 1)
        assert ((got >> 1) & 1) == oracle.orc_check_map(direction, 2)


# ---- window arithmetic ----------------------------------------------------------------
def test_window_arithmetic_equals_oracle(lib, oracle):
    rng = np.random.default_rng(11)
    for _ in range(3000):
        base = int(rng.integers(1, 1 << 40)) * 4096
        stride = int(rng.integers(1, 1 << 20)) * 4096
        ranks = int(rng.integers(1, 9))
        space = int(rng.integers(1, stride // 4096 + 1)) * 4096
        addr = base + int(rng.integers(-5000, stride * ranks + 5000))
        size = int(rng.choice([0, 1, 4096, stride]))
        assert lib.mf_gva_contains(base, stride, ranks, addr, size) == \
            oracle.orc_gva_contains(base, stride, ranks, addr, size)
        assert lib.mf_gva_rank(base, stride, ranks, space, addr) == oracle.orc_gva_rank(base, stride, ranks, space, addr)
    assert lib.mf_gva_contains(0, 4096, 1, 4096, 1) == 0
    for a in (0, 0xFFFF_0000_0000_1234, 2**64 - 1):
        assert lib.mf_gva_mask48(a) == oracle.orc_mask48(a)


# ---- work decomposition ------------------------------------------------------------------
def _describe(lib, src, dst, lens, units):
    n = len(lens)
    cap = 64
    while True:
        out = (ctypes.c_uint64 * (4 * cap))()
        inline = ctypes.c_int32(-1)
        got = lib.mf_xcopy_describe_plan(u64_array(src), u64_array(dst), u64_array(lens), n, units, out, cap,
                                         ctypes.byref(inline))
        if got >= 0:
            ranges = [(out[4 * i], out[4 * i + 1], out[4 * i + 2], out[4 * i + 3]) for i in range(got)]
            return ranges, inline.value
        cap = -got


def _run_plan_on_cpu(ranges, base_src, src_buf, base_dst, dst_buf):
    hits = np.zeros(len(dst_buf), dtype=np.uint8)
    for s, d, l, _ in ranges:
        dst_buf[d - base_dst:d - base_dst + l] = src_buf[s - base_src:s - base_src + l]
        hits[d - base_dst:d - base_dst + l] += 1
    return hits


def test_plan_tiles_every_length_and_alignment(lib, oracle):
    """Lengths 0..257 at every source/destination misalignment: the chunks' byte ranges cover each
    destination byte exactly once and reproduce memcpy."""
    rng = np.random.default_rng(12)
    src_buf = rng.integers(0, 256, 1024, dtype=np.uint8)
    base_src, base_dst = 0x10000, 0x90000
    for length in list(range(0, 258)):
        for sa in (0, 1, 7, 15):
            for da in (0, 3, 8, 15):
                dst_buf = np.full(1024, 0xEE, dtype=np.uint8)
                ranges, inline = _describe(lib, [base_src + sa], [base_dst + da + 32], [length], 256)
                assert inline == 1
                hits = _run_plan_on_cpu(ranges, base_src, src_buf, base_dst, dst_buf)
                expect = np.full(1024, 0xEE, dtype=np.uint8)
                expect[da + 32:da + 32 + length] = src_buf[sa:sa + length]
                assert np.array_equal(dst_buf, expect), (length, sa, da)
                assert hits.max(initial=0) <= 1
                # 16-byte body ranges are destination-aligned
                for s, d, l, _ in ranges:
                    if l >= 16:
                        assert d % 16 == 0 and l % 16 == 0


@pytest.mark.parametrize("units", [256, 512, 1024, 4096])
def test_plan_of_kv_batch_is_balanced_and_exact(lib, oracle, units):
    src, dst, lens = workloads.kv_batch(0xC1, 1 << 28)
    base = 0x7000_0000_0000
    ranges, inline = _describe(lib, base + src, base + dst, lens, units)
    assert inline == 1
    assert sum(r[2] for r in ranges) == workloads.KV_PAYLOAD
    per_chunk = {}
    for _, _, l, c in ranges:
        per_chunk[c] = per_chunk.get(c, 0) + l
    assert max(per_chunk.values()) == min(units * 16, 128 * 1024)
    expected_chunks = sum(max(1, -(-int(l) // (units * 16))) for l in lens)
    assert len(per_chunk) == expected_chunks
    # every destination byte written once
    covered = sorted((d, d + l) for _, d, l, _ in ranges)
    for (a0, a1), (b0, b1) in zip(covered, covered[1:]):
        assert a1 <= b0


def test_plan_of_ragged_batch_reproduces_oracle_copy(lib, oracle):
    pool = 1 << 22
    rng = np.random.default_rng(13)
    src_buf = rng.integers(0, 256, pool, dtype=np.uint8)
    for count, units in [(5, 256), (128, 256), (129, 512), (700, 1024)]:
        so, do, lens = workloads.ragged_batch(100 + count, pool, count, max_len=9000)
        base_src, base_dst = 0x1000_0000, 0x9000_0000
        ranges, inline = _describe(lib, base_src + so, base_dst + do, lens, units)
        assert inline == (1 if np.count_nonzero(lens) <= 128 else 0)
        got = np.full(pool, 0x5A, dtype=np.uint8)
        hits = _run_plan_on_cpu(ranges, base_src, src_buf, base_dst, got)
        assert hits.max() <= 1
        expect = np.full(pool, 0x5A, dtype=np.uint8)
        srcs = ptr_array([np_ptr(src_buf) + int(s) for s in so])
        dsts = ptr_array([np_ptr(expect) + int(d) for d in do])
        assert oracle.orc_batch_copy(dsts, srcs, u64_array(lens), count) == 0
        assert np.array_equal(got, expect)


def test_plan_merges_adjacent_segments_like_the_reference(lib, oracle):
    # 8 pages that continue each other on both sides + 1 stray one
    src = [0x100000 + i * 4096 for i in range(8)] + [0x900000]
    dst = [0x500000 + i * 4096 for i in range(8)] + [0xA00000]
    lens = [4096] * 9
    out = (ctypes.c_uint64 * 27)()
    k = oracle.orc_coalesce(u64_array(src), u64_array(dst), u64_array(lens), 9, out)
    assert k == 2
    ranges, _ = _describe(lib, src, dst, lens, 4096)
    assert sorted((r[0], r[1], r[2]) for r in ranges) == sorted((out[3 * i], out[3 * i + 1], out[3 * i + 2])
                                                               for i in range(k))


def test_plan_splits_segments_the_inline_form_cannot_hold(lib):
    ranges, inline = _describe(lib, [0x1_0000_0000], [0x9_0000_0000], [5 << 30], 4096)
    assert inline == 1
    assert sum(r[2] for r in ranges) == 5 << 30
    assert max(r[2] for r in ranges) == 4096 * 16


def test_choose_units_policy(lib):
    # HBM routes: 4 KiB chunks (single-wave workgroups) at every size; link routes: their own small chunks
    assert lib.mf_xcopy_choose_units(64 * 1024, 256, native.ROUTE_HBM) == 256
    assert lib.mf_xcopy_choose_units(workloads.KV_PAYLOAD, 256, native.ROUTE_HBM) == 256
    assert lib.mf_xcopy_choose_units(1 << 30, 256, native.ROUTE_HBM) == 256
    assert lib.mf_xcopy_choose_units(2 << 30, 256, native.ROUTE_HBM) == 256
    assert lib.mf_xcopy_choose_units(workloads.KV_PAYLOAD, 256, native.ROUTE_TO_HOST) == 256
    assert lib.mf_xcopy_choose_units(workloads.KV_PAYLOAD, 256, native.ROUTE_FROM_HOST) == 512
    assert lib.mf_xcopy_choose_units(1 << 30, 256, native.ROUTE_FROM_HOST) == 1024


# ---- error contracts that need no GPU (test/ut/testcase/smem/smem_bm_test.cpp:59-201 of the reference) ----
def test_config_init_defaults(lib):
    cfg = native.SmemBmConfig()
    assert lib.smem_bm_config_init(ctypes.byref(cfg)) == native.SM_OK
    assert (cfg.initTimeout, cfg.createTimeout, cfg.controlOperationTimeout) == (120, 120, 120)
    assert cfg.startConfigStoreServer and not cfg.startConfigStoreOnly and not cfg.dynamicWorldSize
    assert cfg.unifiedAddressSpace and cfg.autoRanking and cfg.flags == 0 and cfg.rankId == 0xFFFF
    assert lib.smem_bm_config_init(None) == native.SM_INVALID_PARAM


def test_init_argument_checks(lib):
    cfg = native.SmemBmConfig()
    lib.smem_bm_config_init(ctypes.byref(cfg))
    assert lib.smem_bm_init(b"tcp://127.0.0.1:1", 0, 0, ctypes.byref(cfg)) == native.SM_INVALID_PARAM
    assert lib.smem_bm_init(b"tcp://127.0.0.1:1", 1025, 0, ctypes.byref(cfg)) == native.SM_INVALID_PARAM
    assert lib.smem_bm_init(None, 1, 0, ctypes.byref(cfg)) == native.SM_INVALID_PARAM
    assert lib.smem_bm_init(b"tcp://127.0.0.1:1", 1, 0, None) == native.SM_INVALID_PARAM
    bad = native.SmemBmConfig()
    lib.smem_bm_config_init(ctypes.byref(bad))
    bad.unifiedAddressSpace = False
    assert lib.smem_bm_init(b"tcp://127.0.0.1:1", 1, 0, ctypes.byref(bad)) == native.SM_INVALID_PARAM
    bad.unifiedAddressSpace = True
    bad.initTimeout = 0
    assert lib.smem_bm_init(b"tcp://127.0.0.1:1", 1, 0, ctypes.byref(bad)) == native.SM_INVALID_PARAM


def test_calls_before_init(lib):
    fake = ctypes.c_void_p(1)
    params = native.SmemCopyParams(None, None, 0)
    batch = native.BatchCopyParams()
    G2G = native.SMEMB_COPY["G2G"]
    assert lib.smem_bm_create(0, 1, 1, 1 << 21, 1 << 21, 0) is None
    assert lib.smem_bm_create2(0, None) is None
    assert lib.smem_bm_get_local_mem_size_by_mem_type(None, native.SMEM_MEM_TYPE_HOST) == 0
    assert lib.smem_bm_ptr_by_mem_type(None, native.SMEM_MEM_TYPE_HOST, 0) is None
    assert lib.smem_bm_ptr_by_mem_type(fake, native.SMEM_MEM_TYPE_HOST, 0) is None
    assert lib.smem_bm_copy(None, ctypes.byref(params), G2G, 0) == native.SM_INVALID_PARAM
    assert lib.smem_bm_copy(fake, None, G2G, 0) == native.SM_INVALID_PARAM
    assert lib.smem_bm_copy(fake, ctypes.byref(params), G2G, 0) == native.SM_NOT_INITIALIZED
    assert lib.smem_bm_copy_batch(None, ctypes.byref(batch), G2G, 0) == native.SM_INVALID_PARAM
    assert lib.smem_bm_copy_batch(fake, None, G2G, 0) == native.SM_INVALID_PARAM
    assert lib.smem_bm_copy_batch(fake, ctypes.byref(batch), G2G, 0) == native.SM_NOT_INITIALIZED
    assert lib.smem_bm_wait(None) == native.SM_INVALID_PARAM
    assert lib.smem_bm_wait(fake) == native.SM_NOT_INITIALIZED
    assert lib.smem_bm_get_rank_id_by_gva(None, None) == native.SM_INVALID_PARAM & 0xFFFFFFFF
    assert lib.smem_bm_get_rank_id_by_gva(fake, None) == native.SM_NOT_INITIALIZED & 0xFFFFFFFF
    assert lib.smem_bm_register_user_mem(None, 0x1000, 1024) == native.SM_INVALID_PARAM
    assert lib.smem_bm_register_user_mem(fake, 0, 1024) == native.SM_INVALID_PARAM
    assert lib.smem_bm_register_user_mem(fake, 0x1000, 1024) == native.SM_NOT_INITIALIZED
    assert lib.smem_bm_unregister_user_mem(None, 0x1000) == native.SM_INVALID_PARAM
    assert lib.smem_bm_unregister_user_mem(fake, 0) == native.SM_INVALID_PARAM
    assert lib.smem_bm_unregister_user_mem(fake, 0x1000) == native.SM_NOT_INITIALIZED
    assert lib.smem_bm_join(None, 0) == native.SM_INVALID_PARAM
    assert lib.smem_bm_join(fake, 0) == native.SM_NOT_INITIALIZED
    assert lib.smem_bm_get_rank_id() == 0xFFFFFFFF
    lib.smem_bm_uninit(0)  # harmless
    lib.smem_bm_destroy(None)
    assert b"not initialized" in lib.smem_get_last_err_msg()


def test_hybm_argument_checks(lib):
    fake = ctypes.c_void_p(1)
    one = ctypes.c_void_p(0x1000)
    cp = native.HybmCopyParams(0x1000, 0x2000, 16)
    GD2GD = native.HYBM_DIR["GD2GD"]
    assert lib.hybm_data_copy(None, ctypes.byref(cp), GD2GD, None, 0) == native.BM_INVALID_PARAM
    assert lib.hybm_data_copy(fake, None, GD2GD, None, 0) == native.BM_INVALID_PARAM
    assert lib.hybm_data_copy(fake, ctypes.byref(native.HybmCopyParams(0, 0x2000, 16)), GD2GD, None, 0) == -2
    assert lib.hybm_data_copy(fake, ctypes.byref(native.HybmCopyParams(0x1000, 0, 16)), GD2GD, None, 0) == -2
    assert lib.hybm_data_copy(fake, ctypes.byref(native.HybmCopyParams(0x1000, 0x2000, 0)), GD2GD, None, 0) == -2
    assert lib.hybm_data_copy(fake, ctypes.byref(cp), native.HYBM_DIR["BUTT"], None, 0) == native.BM_INVALID_PARAM
    assert lib.hybm_data_copy(fake, ctypes.byref(cp), GD2GD, None, 0) == native.BM_INVALID_PARAM  # unknown handle
    # AUTO with two addresses outside every pool cannot be inferred
    lib.mf_va_clear()
    assert lib.hybm_data_copy(fake, ctypes.byref(cp), native.HYBM_DIR["AUTO"], None, 0) == native.BM_INVALID_PARAM
    srcs = ptr_array([0x1000])
    dsts = ptr_array([0x2000])
    lens = u64_array([16])
    bp = native.BatchCopyParams(srcs, dsts, lens, 1)
    assert lib.hybm_data_batch_copy(None, ctypes.byref(bp), GD2GD, None, 0) == native.BM_INVALID_PARAM
    assert lib.hybm_data_batch_copy(fake, None, GD2GD, None, 0) == native.BM_INVALID_PARAM
    assert lib.hybm_data_batch_copy(fake, ctypes.byref(native.BatchCopyParams(None, dsts, lens, 1)), GD2GD, None, 0) == -2
    assert lib.hybm_data_batch_copy(fake, ctypes.byref(native.BatchCopyParams(srcs, None, lens, 1)), GD2GD, None, 0) == -2
    assert lib.hybm_data_batch_copy(fake, ctypes.byref(native.BatchCopyParams(srcs, dsts, None, 1)), GD2GD, None, 0) == -2
    assert lib.hybm_data_batch_copy(fake, ctypes.byref(native.BatchCopyParams(srcs, dsts, lens, 0)), GD2GD, None, 0) == -2
    assert lib.hybm_data_batch_copy(fake, ctypes.byref(bp), 13, None, 0) == native.BM_INVALID_PARAM
    assert lib.hybm_wait(None) == native.BM_INVALID_PARAM
    assert lib.hybm_create_entity(1, None, 0) is None
    assert lib.hybm_set_log_level(7) == native.BM_INVALID_PARAM
    assert lib.hybm_set_log_level(2) == native.BM_OK


def test_product_fails_loudly_without_a_gpu_runtime(lib):
    """Raw enqueue before any init: an error code, never a silent CPU copy."""
    if lib.mfrt_is_initialised():
        pytest.skip("runtime already initialised in this process")
    a = np.arange(64, dtype=np.uint8)
    b = np.zeros(64, dtype=np.uint8)
    ret = lib.mf_xcopy_batch(u64_array([np_ptr(a)]), u64_array([np_ptr(b)]), u64_array([64]), 1, 0, None)
    assert ret == native.BM_NOT_INITIALIZED
    assert not b.any()


def test_workload_generators():
    src, dst, lens = workloads.kv_batch(0xC1, 4 << 30)
    assert len(lens) == 122 and int(lens.sum()) == workloads.KV_PAYLOAD == 8994816
    assert np.all(src % 4096 == 0) and np.all(dst % 4096 == 0)
    iv = sorted([(int(d), int(d + l)) for d, l in zip(dst, lens)] + [(int(s), int(s + l)) for s, l in zip(src, lens)])
    for (a0, a1), (b0, b1) in zip(iv, iv[1:]):
        assert a1 <= b0
    src2, dst2, _ = workloads.kv_batch(0xC1, 4 << 30)
    assert np.array_equal(src, src2) and np.array_equal(dst, dst2)
    src3, _, _ = workloads.kv_batch(0xC2, 4 << 30)
    assert not np.array_equal(src, src3)
    ids = workloads.page_ids(0xC3, 1310720, 4096)
    assert len(set(ids.tolist())) == 4096


# ---- 2-D copy: index arithmetic of the kernel ---------------------------------------------------
def test_2d_row_and_column_of_every_unit_in_a_chunk(lib):
    """For every row width the planner can produce, the kernel's (row, column) of each 16-byte unit
    of a chunk equals u // widthUnits, u % widthUnits.  Chunks of several rows use a multiply-high
    division; a chunk that holds one row must not (the multiply-high is wrong from 65 537 units on:
    unit 65 536 of such a row would land in "row 1, column 2^32 - 1")."""
    widths = list(range(1, 1100)) + [4095, 4096, 4097, 65535, 65536, 65537, (1 << 20) - 1, 1 << 20, (1 << 20) + 1,
                                     131073, (1 << 24) + 3]
    rng = np.random.default_rng(5)
    widths += [int(v) for v in rng.integers(2, 1 << 20, 200)]
    for wu in widths:
        rpc, magic = ctypes.c_uint32(0), ctypes.c_uint32(0)
        lib.mf_copy2d_describe(wu * 16, ctypes.byref(rpc), ctypes.byref(magic))
        assert rpc.value == max(1, 16384 // (wu * 16))
        units = rpc.value * wu
        assert lib.mf_copy2d_rowcol_mismatches(wu, rpc.value, magic.value, units) == 0, wu
    # the formula the one-row case must not use: the multiply-high alone, on a row of 65 537 units
    assert lib.mf_copy2d_rowcol_mismatches(65537, 2, (1 << 32) // 65537 + 1, 65537) != 0


def test_python_side_knows_the_combine_pace_the_library_starts_with():
    """bench.py and the GPU tests switch the windowed combine off and back on with native.MOE_COMBINE_WINDOWS_DEFAULT."""
    import pathlib
    import re
    text = (pathlib.Path(native.__file__).parent / "csrc" / "kernels" / "moe.hip").read_text()
    read = int(re.search(r"g_combineReadMBps\{(\d+)\}", text).group(1))
    write = int(re.search(r"g_combineWriteMBps\{(\d+)\}", text).group(1))
    assert (read, write) == native.MOE_COMBINE_WINDOWS_DEFAULT
