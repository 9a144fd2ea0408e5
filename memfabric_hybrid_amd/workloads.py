"""Synthetic inputs of the benchmark configurations (host side, numpy only).

Segment tables are reproducible functions of a seed; payload bytes are filled
by the caller (tests use the oracle's splitmix64 stream, the benchmark fills
pools on the GPU).  Sizes follow the workload definitions:

* KV block batch: 61 x (128 KiB, 16 KiB) = 122 segments, 8 994 816 bytes,
  4 KiB aligned offsets inside one pool, no destination overlapping another
  destination or any source (copies of a batch run concurrently).
* paged KV gather/scatter: 4096 distinct 32 KiB pages.
* 7B reshard TP8 -> TP4: contiguous column-parallel merges and 2-D strided
  row-parallel merges.
"""

import numpy as np

KV_LAYERS = 61
KV_K_BYTES = 128 * 1024
KV_V_BYTES = 16 * 1024
KV_SEGMENTS = 2 * KV_LAYERS
KV_PAYLOAD = KV_LAYERS * (KV_K_BYTES + KV_V_BYTES)  # 8 994 816
SLOT = 4096


def kv_sizes():
    sizes = np.empty(KV_SEGMENTS, dtype=np.uint64)
    sizes[0::2] = KV_K_BYTES
    sizes[1::2] = KV_V_BYTES
    return sizes


def _place(rng, sizes, pool_bytes, taken, align=SLOT, max_tries=10000):
    """Rejection-sample an aligned offset for each size avoiding every interval in `taken`.

    Meant for sparse placements (a few hundred ranges in a pool many times their total);
    raises instead of spinning when the pool is too full for that.
    """
    offs = np.empty(len(sizes), dtype=np.uint64)
    slots = pool_bytes // align
    for i, size in enumerate(sizes):
        size = int(size)
        need = (size + align - 1) // align
        for _ in range(max_tries):
            start = int(rng.integers(0, slots - need + 1)) * align
            end = start + size
            if all(end <= a or start >= b for a, b in taken):
                break
        else:
            raise ValueError("pool too full for random placement")
        taken.append((start, end))
        offs[i] = start
    return offs


def _pack(rng, sizes, region_start, region_bytes, align):
    """Disjoint offsets inside [region_start, +region_bytes): ranges laid end to end in a random
    order with random gaps.  Always terminates; raises if the region is too small."""
    n = len(sizes)
    padded = [(int(s) + align - 1) // align * align for s in sizes]
    slack = region_bytes - sum(padded)
    if slack < 0:
        raise ValueError("region too small for the requested ranges")
    gaps = rng.multinomial(slack // align, np.full(n + 1, 1.0 / (n + 1)))[:n] * align
    order = rng.permutation(n)
    offs = np.empty(n, dtype=np.uint64)
    cursor = region_start
    for j, i in enumerate(order):
        cursor += int(gaps[j])
        offs[i] = cursor
        cursor += padded[i]
    return offs


def kv_batch(seed, src_pool_bytes, dst_pool_bytes=None, same_pool=True, sizes=None):
    """Offsets (src, dst, len) of one 122-segment batch.

    same_pool: sources and destinations share one pool (device to device inside the HBM
    pool), so sources must avoid destinations too; otherwise the two sides live in
    different pools and only destinations must be pairwise disjoint.
    """
    rng = np.random.default_rng(seed)
    sizes = kv_sizes() if sizes is None else np.asarray(sizes, dtype=np.uint64)
    dst_pool_bytes = src_pool_bytes if dst_pool_bytes is None else dst_pool_bytes
    taken = []
    dst = _place(rng, sizes, dst_pool_bytes, taken)
    if same_pool:
        src = _place(rng, sizes, src_pool_bytes, taken)  # disjoint from all destinations (and other sources)
    else:
        src = _place(rng, sizes, src_pool_bytes, [])
    return src, dst, sizes.copy()


def ragged_batch(seed, pool_bytes, count, max_len=70000, align=1):
    """Arbitrary byte lengths (including 0) at arbitrary byte offsets; sources in the lower
    half of the pool, destinations (pairwise disjoint) in the upper half."""
    rng = np.random.default_rng(seed)
    sizes = rng.integers(0, max_len + 1, size=count).astype(np.uint64)
    sizes[rng.integers(0, count, size=max(1, count // 8))] = 0
    small = rng.integers(0, count, size=max(1, count // 4))
    sizes[small] = rng.integers(0, 40, size=len(small)).astype(np.uint64)
    half = pool_bytes // 2
    budget = half - count * max(align, 1)
    while int(sizes.sum()) > budget:  # shrink deterministically until both halves can hold the batch
        sizes //= 2
    src = _pack(rng, sizes, 0, half, align)
    dst = _pack(rng, sizes, half, half, align)
    return src, dst, sizes


def page_ids(seed, total_pages, count):
    rng = np.random.default_rng(seed)
    return rng.choice(total_pages, size=count, replace=False).astype(np.uint64)


def moe_inputs(seed, tokens, hidden, experts, topk):
    """bf16 N(0,1) activations as uint16 words, fp32 N(0,1) router logits."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((tokens, hidden), dtype=np.float32)
    logits = rng.standard_normal((tokens, experts), dtype=np.float32)
    return f32_to_bf16_words(x), logits


def f32_to_bf16_words(a):
    w = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    bias = np.uint32(0x7FFF) + ((w >> np.uint32(16)) & np.uint32(1))
    return ((w + bias) >> np.uint32(16)).astype(np.uint16)


def bf16_words_to_f32(w):
    return (w.astype(np.uint32) << np.uint32(16)).view(np.float32)


# ---- 7B decoder reshard, TP=8 storage -> TP=4 layout -------------------------
RESHARD_LAYERS = 28
RESHARD_HIDDEN = 3584
RESHARD_FFN = 18944
RESHARD_KV_OUT = 512  # 4 KV heads x 128


def reshard_tensors():
    """(name, rows(out), cols(in), kind) of one layer; kind 'col' splits rows, 'row' splits columns."""
    h, f, kv = RESHARD_HIDDEN, RESHARD_FFN, RESHARD_KV_OUT
    return [
        ("q", h, h, "col"), ("k", kv, h, "col_kv"), ("v", kv, h, "col_kv"), ("o", h, h, "row"),
        ("gate", f, h, "col"), ("up", f, h, "col"), ("down", h, f, "row"),
    ]
