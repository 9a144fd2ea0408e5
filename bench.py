#!/usr/bin/env python3
"""Benchmark of the 122-segment KV-block batch copy (device to device inside a 4 GiB HBM pool)
through smem_bm_copy_batch, plus the CPU baseline and the roofline of the copy kernel.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--extras]

A step is one batch: 61 x (128 KiB + 16 KiB) = 8 994 816 payload bytes, i.e. 17 989 632 bytes
of HBM traffic (read + write).  Steps rotate over 64 different segment tables so that the
touched set (about 1.1 GiB) does not fit the 256 MiB last-level cache.  Prints one JSON line.
"""

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from memfabric_hybrid_amd import bm, native, workloads  # noqa: E402

GB = 1e9
HBM_PEAK_GBPS = 8000.0
LINK_PEAK_GBPS = 64.0
POOL_BYTES = 4 << 30
TABLES = 64


class Batch:
    """One segment table in the exact form smem_bm_copy_batch takes."""

    def __init__(self, src, dst, lens):
        self.n = len(lens)
        self.srcs = native.ptr_array(src.tolist())
        self.dsts = native.ptr_array(dst.tolist())
        self.lens = native.u64_array(lens.tolist())
        self.params = native.BatchCopyParams(self.srcs, self.dsts, self.lens, self.n)
        self.ref = ctypes.byref(self.params)
        self.payload = int(lens.sum())


def fill_device_pool(lib, dev, nbytes, seed):
    """Uniform random bytes: a 64 MiB block generated on the host, uploaded and re-uploaded with a
    different XOR mask per block so that no two blocks are equal."""
    rng = np.random.default_rng(seed)
    block = rng.integers(0, 256, 64 << 20, dtype=np.uint8)
    for i in range(nbytes // len(block)):
        chunk = block ^ np.uint8((i * 37 + 11) & 0xFF)
        err = lib.mfrt_memcpy(dev + i * len(block), chunk.ctypes.data, len(block))
        assert err == 0, lib.mfrt_error_string(err)


def timed_steps(lib, handle, batches, copy_type, steps, warmup, flags):
    """K async batch copies between two events on the launch stream; returns (wall s, event ms)."""
    stream = lib.mf_xcopy_thread_stream()
    start, stop = lib.mfrt_event_create(), lib.mfrt_event_create()
    call = lib.smem_bm_copy_batch
    nb = len(batches)
    for i in range(warmup):
        ret = call(handle, batches[i % nb].ref, copy_type, flags)
        assert ret == 0, native.last_error()
    assert lib.mfrt_stream_sync(stream) == 0
    assert lib.mfrt_device_sync() == 0
    t0 = time.perf_counter()
    lib.mfrt_event_record(start, stream)
    for i in range(steps):
        ret = call(handle, batches[i % nb].ref, copy_type, flags)
        if ret != 0:
            raise RuntimeError(native.last_error())
    lib.mfrt_event_record(stop, stream)
    assert lib.mfrt_stream_sync(stream) == 0
    assert lib.mfrt_device_sync() == 0
    wall = time.perf_counter() - t0
    ms = lib.mfrt_event_elapsed_ms(start, stop)
    lib.mfrt_event_destroy(start)
    lib.mfrt_event_destroy(stop)
    return wall, ms


def cpu_baseline(tables, budget_s=12.0):
    """The reference's CPU copy path (single thread, one memcpy per segment, host pool to host
    pool) on the same segment tables: the reference's own DlHybridApi::Memcpy when oracle/_ref was
    built, else the oracle's restatement of it."""
    from tests import oracle_lib
    ref = oracle_lib.reference()
    fn = ref.ref_batch_copy if ref is not None else oracle_lib.oracle().orc_batch_copy_fast
    kind = "reference" if ref is not None else "port"
    pool = 1 << 30  # host pools of 1 GiB each; the tables are folded into them
    src_pool = np.random.default_rng(1).integers(0, 256, pool, dtype=np.uint8)
    dst_pool = np.zeros(pool, dtype=np.uint8)
    prepared = []
    for src, dst, lens in tables:
        s = oracle_lib.ptr_array((src_pool.ctypes.data + (src % np.uint64(pool - (1 << 20)))).tolist())
        d = oracle_lib.ptr_array((dst_pool.ctypes.data + (dst % np.uint64(pool - (1 << 20)))).tolist())
        prepared.append((d, s, oracle_lib.u64_array(lens.tolist()), len(lens), int(lens.sum())))
    for d, s, l, n, _ in prepared[:8]:
        fn(d, s, l, n)
    done_bytes, batches, t0 = 0, 0, time.perf_counter()
    while True:
        for d, s, l, n, payload in prepared:
            fn(d, s, l, n)
            done_bytes += payload
            batches += 1
        elapsed = time.perf_counter() - t0
        if elapsed > budget_s or batches >= 64 * 40:
            break
    return {
        "value": done_bytes / elapsed / GB,
        "unit": "GB/s payload",
        "cores": 1,
        "kind": kind,
        "sample": f"{batches} batches of the same 122-segment tables, host pool to host pool, "
                  f"{elapsed:.1f} s, single thread, nproc={os.cpu_count()}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=400)
    ap.add_argument("--extras", action="store_true", help="also time H2D / D2H and synchronous calls")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is a single-GPU data plane (no collectives, no sharding); run with --gpus 1")

    lib = native.lib()
    assert bm.initialize("tcp://127.0.0.1:0", 1, 0) == 0, native.last_error()
    want_host = POOL_BYTES if args.extras else 0
    pool = bm.create(0, want_host, POOL_BYTES)
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    fill_device_pool(lib, dev, POOL_BYTES, 0xC1)

    tables = [workloads.kv_batch(0xC1 + b, POOL_BYTES) for b in range(TABLES)]
    batches = [Batch(dev + s, dev + d, l) for s, d, l in tables]
    payload = batches[0].payload
    g2g = int(bm.BmCopyType.G2G)

    wall, ms = timed_steps(lib, pool.handle, batches, g2g, args.steps, args.warmup, native.ASYNC_COPY_FLAG)
    per_launch_us = ms * 1e3 / args.steps
    value = payload * args.steps / wall / GB
    achieved = 2 * payload / (per_launch_us * 1e-6) / GB

    result = {
        "metric": "achieved GB/s (payload) for 122-segment KV batch copy, device to device",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall * 1e3 / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {
            "workload": "DeepSeek-R1-style KV block batch: 122 segments (61x128KiB + 61x16KiB = 8994816 B), "
                        "4 KiB-aligned random offsets in a 4 GiB HBM pool, D2D, 64 rotating tables",
            "api": "smem_bm_copy_batch(SMEMB_COPY_G2G, ASYNC_COPY_FLAG) + one wait",
            "payload_bytes": payload,
            "cu_count": lib.mfrt_cu_count(),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": None,
            "kernel": "XcopyInlineKernel<HBM>",
            "algorithmic_bytes_per_launch": 2 * payload,
            "avg_launch_us": per_launch_us,
        },
    }

    if args.extras:
        extras = {}
        w2, m2 = timed_steps(lib, pool.handle, batches, g2g, max(200, args.steps // 10), 50, 0)
        extras["d2d_sync_call_us"] = w2 * 1e6 / max(200, args.steps // 10)
        host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
        split = [workloads.kv_batch(0xD1 + b, POOL_BYTES, same_pool=False) for b in range(TABLES)]
        h2d = [Batch(host + s, dev + d, l) for s, d, l in split]
        d2h = [Batch(dev + s, host + d, l) for s, d, l in split]
        for name, bs in (("h2d", h2d), ("d2h", d2h)):
            k = max(100, args.steps // 20)
            w, m = timed_steps(lib, pool.handle, bs, g2g, k, 20, native.ASYNC_COPY_FLAG)
            gbps = payload * k / (m * 1e-3) / GB
            extras[name] = {"GBps": gbps, "frac_of_link_peak": gbps / LINK_PEAK_GBPS, "us_per_batch": m * 1e3 / k}
        result["extras"] = extras

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(tables)

    pool.destroy()
    bm.uninitialize()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
