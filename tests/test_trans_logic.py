"""Arithmetic of the transfer front-end, CPU only: the oracle's restatement of
SmemTransEntry::AlignMemory / CombineMemories and of the remote-address lookup
(src/smem/csrc/smem_trans/smem_trans_entry.cpp:337-356,604-640 of the reference) pinned by closed
forms and brute force, then the library's own versions compared with the oracle.  The reference's
unit tests for this layer need two processes and a config store and hold no vectors for it."""

import ctypes

import numpy as np
import pytest

from memfabric_hybrid_amd import native
from tests.oracle_lib import np_ptr

PAGE = 2 << 20
u64p = ctypes.POINTER(ctypes.c_uint64)


def _u64(a):
    return a.ctypes.data_as(u64p)


def _oracle_align(oracle, addr, size):
    a, s = ctypes.c_uint64(addr), ctypes.c_uint64(size)
    oracle.orc_trans_align(ctypes.byref(a), ctypes.byref(s))
    return a.value, s.value


def test_oracle_page_hull_is_the_minimal_aligned_cover(oracle):
    rng = np.random.default_rng(0xA11)
    cases = [(PAGE, PAGE), (PAGE, 1), (PAGE - 1, 2), (PAGE + 1, PAGE - 1), (5 * PAGE + 7, 3 * PAGE), (1, 1)]
    cases += [(int(rng.integers(1, 1 << 44)), int(rng.integers(1, 1 << 30))) for _ in range(2000)]
    for addr, size in cases:
        start, length = _oracle_align(oracle, addr, size)
        assert start % PAGE == 0 and length % PAGE == 0 and length > 0
        assert start <= addr and addr + size <= start + length          # covers
        assert start + PAGE > addr                                      # a later start would uncover the first byte
        assert start + length - PAGE < addr + size                      # a shorter hull would uncover the last byte


def _union_by_bitmap(pairs, span):
    """Brute force: mark every unit of every range, then read maximal runs back.  Ranges that
    merely touch also merge, which the bitmap cannot see, so touching is tracked separately:
    unit i carries a 'joined to i+1' flag whenever some range covers both or one range ends where
    another starts."""
    covered = np.zeros(span + 1, dtype=bool)
    glued = np.zeros(span + 1, dtype=bool)      # glued[i]: position i is interior to a range or a range start met by an end
    starts = {s for s, _ in pairs}
    for s, n in pairs:
        covered[s:s + n] = True
        glued[s + 1:s + n] = True
        if s + n in starts:
            glued[s + n] = True
    runs = []
    i = 0
    while i < span:
        if not covered[i]:
            i += 1
            continue
        j = i + 1
        while j < span and covered[j] and glued[j]:
            j += 1
        runs.append((i, j - i))
        i = j
    return runs


def test_oracle_combine_equals_brute_force_union(oracle):
    rng = np.random.default_rng(0xC0B)
    for trial in range(400):
        n = int(rng.integers(1, 9))
        pairs = [(int(rng.integers(0, 48)), int(rng.integers(1, 12))) for _ in range(n)]
        flat = np.array([v for p in pairs for v in p], dtype=np.uint64)
        out = np.zeros(2 * n, dtype=np.uint64)
        k = oracle.orc_trans_combine(_u64(flat), n, _u64(out))
        got = [(int(out[2 * i]), int(out[2 * i + 1])) for i in range(k)]
        assert got == _union_by_bitmap(pairs, 64), (trial, pairs)


def test_oracle_combine_known_answers(oracle):
    def run(pairs):
        flat = np.array([v for p in pairs for v in p], dtype=np.uint64)
        out = np.zeros(len(flat), dtype=np.uint64)
        k = oracle.orc_trans_combine(_u64(flat), len(pairs), _u64(out))
        return [(int(out[2 * i]), int(out[2 * i + 1])) for i in range(k)]

    assert run([(10, 5)]) == [(10, 5)]
    assert run([(20, 5), (10, 5)]) == [(10, 5), (20, 5)]                 # sorted, disjoint
    assert run([(10, 5), (15, 5)]) == [(10, 10)]                         # touching pieces join
    assert run([(10, 10), (12, 3)]) == [(10, 10)]                        # contained
    assert run([(10, 5), (10, 9), (16, 1)]) == [(10, 9)]                 # same start, longer one wins
    high = (1 << 47) - (1 << 21)
    assert run([(high + 4, 4), (high, 8), (high + 9, 1)]) == [(high, 8), (high + 9, 1)]   # user-space top, one byte gap


def _translate_by_bytes(slices, remote, size):
    """Brute force for disjoint slices: every byte of the range must belong to the slice that owns
    its first byte's predecessor-or-equal start."""
    owner = {}
    for start, length, mapped in slices:
        for b in range(start, start + length):
            owner[b] = (start, mapped)
    candidates = [s for s in slices if s[0] <= remote]
    if not candidates:
        return 0
    start, length, mapped = max(candidates)
    for b in range(remote, remote + size):
        if owner.get(b, (None, None))[0] != start:
            return 0
    if size == 0 and not (start <= remote <= start + length):
        return 0
    return mapped + (remote - start)


def test_oracle_translate_equals_byte_ownership(oracle):
    rng = np.random.default_rng(0x7A)
    for trial in range(300):
        slices, cursor = [], 0
        for _ in range(int(rng.integers(1, 6))):
            cursor += int(rng.integers(0, 6))
            length = int(rng.integers(1, 10))
            slices.append((cursor, length, 1000 * (len(slices) + 1)))
            cursor += length
        order = rng.permutation(len(slices))
        flat = np.array([v for i in order for v in slices[i]], dtype=np.uint64)
        for remote in range(0, cursor + 3):
            for size in range(1, 12):
                got = oracle.orc_trans_translate(_u64(flat), len(slices), remote, size)
                assert got == _translate_by_bytes(slices, remote, size), (trial, slices, remote, size)


def test_library_combine_and_translate_match_oracle(oracle):
    lib = native.lib()
    rng = np.random.default_rng(0x11B)
    for trial in range(500):
        n = int(rng.integers(1, 40))
        scale = int(rng.choice([64, 1 << 20, 1 << 40]))
        pairs = np.empty(2 * n, dtype=np.uint64)
        pairs[0::2] = rng.integers(1, scale, n)
        pairs[1::2] = rng.integers(1, max(2, scale // 8), n)
        if trial % 3 == 0 and n > 1:                     # force exact touches and duplicates
            pairs[2] = pairs[0] + pairs[1]
            pairs[2 * (n - 1)] = pairs[0]
        want = np.zeros(2 * n, dtype=np.uint64)
        k = oracle.orc_trans_combine(_u64(pairs.copy()), n, _u64(want))
        got = np.zeros(2 * n, dtype=np.uint64)
        assert lib.mf_trans_combine(_u64(pairs), n, _u64(got)) == k
        assert np.array_equal(got[:2 * k], want[:2 * k]), trial
        # the merged runs are disjoint: use them as a slice map and probe around every edge
        slices = np.empty(3 * k, dtype=np.uint64)
        slices[0::3] = want[0:2 * k:2]
        slices[1::3] = want[1:2 * k:2]
        slices[2::3] = want[0:2 * k:2] + np.uint64(1 << 50)
        for i in range(k):
            start, length = int(want[2 * i]), int(want[2 * i + 1])
            for remote in {max(0, start - 1), start, start + length // 2, start + length - 1, start + length}:
                for size in (1, 2, length, length + 1, max(1, start + length - remote)):
                    a = oracle.orc_trans_translate(_u64(slices), k, remote, size)
                    b = lib.mf_trans_translate(_u64(slices), k, remote, size)
                    assert a == b, (trial, start, length, remote, size)


@pytest.mark.parametrize("name,ok", [
    ("127.0.0.1:5321", True), ("10.20.30.40:65535", True), ("[::1]:5321", True), ("[fe80::1]:1", True),
    ("127.0.0.1:1024", False), ("127.0.0.1:80", False), ("127.0.0.1:65536", False), ("0.0.0.0:5321", False),
    ("127.0.0.1", False), ("127.0.0.1:", False), (":5321", False), ("256.1.1.1:5321", False),
    ("[::1]5321", False), ("[::1]:0", False), ("[zz]:5321", False), ("", False), ("127.0.0.1:53a1", False),
])
def test_name_parsing(name, ok):
    """Names the reference's tests use (test/ut/testcase/smem/smem_trans_test.cpp:33-36) and the
    limits of its URL check (src/smem/csrc/net/smem_net_common.cpp:48-96): IPv4 ports must be above
    1024, the address 0.0.0.0 is refused."""
    lib = native.lib()
    key = (ctypes.c_uint8 * 20)()
    assert lib.mf_trans_parse_name(name.encode(), key) == (1 if ok else 0)
    if ok:
        again = (ctypes.c_uint8 * 20)()
        assert lib.mf_trans_parse_name(name.encode(), again) == 1 and bytes(key) == bytes(again)


def test_names_are_distinct_keys():
    lib = native.lib()
    names = ["127.0.0.1:5321", "127.0.0.1:5322", "127.0.0.2:5321", "[::1]:5321", "[::2]:5321", "[::1]:5322"]
    keys = []
    for n in names:
        key = (ctypes.c_uint8 * 20)()
        assert lib.mf_trans_parse_name(n.encode(), key) == 1
        keys.append(bytes(key))
    assert len(set(keys)) == len(names)
