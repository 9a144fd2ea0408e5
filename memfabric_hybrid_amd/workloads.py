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


def moe_route(logits, topk):
    """Top-k experts per token by logit, ties to the lower expert id, and the softmax of the
    selected logits in fp32 (the routing the MoE workload is specified with)."""
    order = np.argsort(-logits, axis=1, kind="stable")[:, :topk].astype(np.int32)
    picked = np.take_along_axis(logits, order, axis=1).astype(np.float32)
    e = np.exp(picked - picked.max(axis=1, keepdims=True), dtype=np.float32)
    return np.ascontiguousarray(order), np.ascontiguousarray(e / e.sum(axis=1, keepdims=True, dtype=np.float32))


def f32_to_bf16_words(a):
    w = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    bias = np.uint32(0x7FFF) + ((w >> np.uint32(16)) & np.uint32(1))
    return ((w + bias) >> np.uint32(16)).astype(np.uint16)


def bf16_words_to_f32(w):
    return (w.astype(np.uint32) << np.uint32(16)).view(np.float32)


# ---- decoder weight reshard, TP=8 storage -> TP=4 layout ---------------------------
# Row-major [out, in] bf16 tensors per layer.  Column-parallel tensors (q, gate, up) are split on
# `out`; k and v (4 KV heads) are split per head, each head held by two of the eight ranks;
# row-parallel tensors (o, down) are split on `in`.
RESHARD_LAYERS = 28
RESHARD_HIDDEN = 3584
RESHARD_FFN = 18944
RESHARD_KV_HEADS = 4
RESHARD_HEAD_DIM = 128
ELEM = 2


def reshard_tensors(hidden=RESHARD_HIDDEN, ffn=RESHARD_FFN, kv_heads=RESHARD_KV_HEADS, head_dim=RESHARD_HEAD_DIM):
    """(name, out rows, in cols, kind) of one layer."""
    kv = kv_heads * head_dim
    return [("q", hidden, hidden, "col"), ("k", kv, hidden, "kv"), ("v", kv, hidden, "kv"),
            ("o", hidden, hidden, "row"), ("gate", ffn, hidden, "col"), ("up", ffn, hidden, "col"),
            ("down", hidden, ffn, "row")]


def tp8_shard_shape(out, cols, kind):
    if kind == "col":
        return out // 8, cols
    if kind == "kv":
        return out // 4, cols          # one KV head per rank, every head on two ranks
    return out, cols // 8


def tp4_shard_shape(out, cols, kind):
    if kind in ("col", "kv"):
        return out // 4, cols
    return out, cols // 4


def reshard_layout(tensors, layers):
    """Byte offsets of every (layer, tensor, shard) in the TP8 source pool and the TP4 destination
    pool, plus the pool sizes.  Shards of a tensor are stored one after another in rank order."""
    src, dst = {}, {}
    s_off = d_off = 0
    for layer in range(layers):
        for name, out, cols, kind in tensors:
            r8, c8 = tp8_shard_shape(out, cols, kind)
            for r in range(8):
                src[(layer, name, r)] = s_off
                s_off += r8 * c8 * ELEM
            r4, c4 = tp4_shard_shape(out, cols, kind)
            for r in range(4):
                dst[(layer, name, r)] = d_off
                d_off += r4 * c4 * ELEM
    return src, dst, s_off, d_off


def reshard_plan(tensors, layers, src_base, dst_base):
    """The re-layout as copy descriptors: (segments, rectangles).

    segments: list of (src, dst, bytes) contiguous copies (column-parallel merges; KV duplicates
    are simply not read).  rectangles: list of (src, dst, width, height, spitch, dpitch) strided
    copies (row-parallel merges: two old column blocks side by side in each new shard)."""
    src, dst, _, _ = reshard_layout(tensors, layers)
    segments, rects = [], []
    for layer in range(layers):
        for name, out, cols, kind in tensors:
            r8, c8 = tp8_shard_shape(out, cols, kind)
            shard_bytes = r8 * c8 * ELEM
            for new in range(4):
                d = dst_base + dst[(layer, name, new)]
                if kind == "col":
                    for half in range(2):
                        segments.append((src_base + src[(layer, name, 2 * new + half)], d + half * shard_bytes,
                                         shard_bytes))
                elif kind == "kv":
                    segments.append((src_base + src[(layer, name, 2 * new)], d, shard_bytes))
                else:
                    width = c8 * ELEM
                    for half in range(2):
                        rects.append((src_base + src[(layer, name, 2 * new + half)], d + half * width, width, out,
                                      width, 2 * width))
    return segments, rects


def reshard_reference(tensors, layers, full):
    """TP8 storage and the expected TP4 storage cut directly out of the full tensors
    full[(layer, name)] (uint16 arrays [out, in]); independent of the descriptors above."""
    src, dst, s_bytes, d_bytes = reshard_layout(tensors, layers)
    s_pool = np.zeros(s_bytes // ELEM, dtype=np.uint16)
    d_pool = np.zeros(d_bytes // ELEM, dtype=np.uint16)
    for layer in range(layers):
        for name, out, cols, kind in tensors:
            w = full[(layer, name)]
            for r in range(8):
                if kind == "col":
                    part = w[r * (out // 8):(r + 1) * (out // 8), :]
                elif kind == "kv":
                    head = r // 2
                    part = w[head * (out // 4):(head + 1) * (out // 4), :]
                else:
                    part = w[:, r * (cols // 8):(r + 1) * (cols // 8)]
                o = src[(layer, name, r)] // ELEM
                s_pool[o:o + part.size] = part.reshape(-1)
            for r in range(4):
                if kind in ("col", "kv"):
                    part = w[r * (out // 4):(r + 1) * (out // 4), :]
                else:
                    part = w[:, r * (cols // 4):(r + 1) * (cols // 4)]
                o = dst[(layer, name, r)] // ELEM
                d_pool[o:o + part.size] = part.reshape(-1)
    return s_pool, d_pool
