#!/usr/bin/env python3
"""Benchmark of the MemFabric xcopy hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu] | --calibrate | --phases [requests ...]
                    | --only paged|reshard|moe

Headline (value / roofline): the 122-segment KV-block batch copy, device to device inside a
4 GiB HBM pool, through smem_bm_copy_batch on one stream.  A step is one batch:
61 x (128 KiB + 16 KiB) = 8 994 816 payload bytes = 17 989 632 bytes of HBM traffic.  Steps
rotate over 64 segment tables so that the touched set (~1.1 GiB) exceeds the 256 MiB
last-level cache.  Whatever --steps and --warmup say, the GPU is first brought to its steady
state by an untimed ramp of RAMP_BATCHES batches; then REPETITIONS repetitions of --steps
batches are timed, each between two synchronisations, and the line reports the median
repetition (HIP events on the launch stream for the kernel rate, the host clock for `value`).  `extras` holds the other workload shapes (host link, large copies, paged
gather, MoE dispatch/combine, weight reshard), concurrency and the yardstick kernels.
Prints ONE JSON line.
"""

import argparse
import ctypes
import json
import os
import sys
import threading
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
MIB = 1 << 20
RAMP_BATCHES = 3000      # untimed, before anything is measured: clocks up, queues and caches in their running state
REPETITIONS = 21         # timed repetitions of --steps batches each; the median is reported
MIN_BATCHES = 2000       # the concurrency extras run at least this many batches per configuration


class Batch:
    """One segment table in the exact form smem_bm_copy_batch takes."""

    def __init__(self, src, dst, lens):
        self.n = len(lens)
        self.srcs = native.ptr_array(np.asarray(src).tolist())
        self.dsts = native.ptr_array(np.asarray(dst).tolist())
        self.lens = native.u64_array(np.asarray(lens).tolist())
        self.params = native.BatchCopyParams(self.srcs, self.dsts, self.lens, self.n)
        self.ref = ctypes.byref(self.params)
        self.payload = int(np.asarray(lens).sum())


class Timer:
    """HIP events on the stream the kernels are launched on."""

    def __init__(self, lib):
        self.lib = lib
        self.stream = lib.mf_xcopy_thread_stream()
        self.e0 = lib.mfrt_event_create()
        self.e1 = lib.mfrt_event_create()

    def run(self, fn, reps, warm=2):
        lib = self.lib
        for _ in range(warm):
            fn()
        assert lib.mfrt_stream_sync(self.stream) == 0
        t0 = time.perf_counter()
        lib.mfrt_event_record(self.e0, self.stream)
        for _ in range(reps):
            fn()
        lib.mfrt_event_record(self.e1, self.stream)
        assert lib.mfrt_stream_sync(self.stream) == 0
        wall = time.perf_counter() - t0
        return lib.mfrt_event_elapsed_ms(self.e0, self.e1) * 1e3 / reps, wall * 1e6 / reps  # us, us


def fill_device_pool(lib, dev, nbytes, seed):
    """Uniform random bytes: a 64 MiB host block, re-uploaded with a different XOR mask per block."""
    rng = np.random.default_rng(seed)
    block = rng.integers(0, 256, 64 * MIB, dtype=np.uint8)
    for i in range(nbytes // len(block)):
        chunk = block ^ np.uint8((i * 37 + 11) & 0xFF)
        err = lib.mfrt_memcpy(dev + i * len(block), chunk.ctypes.data, len(block))
        assert err == 0, lib.mfrt_error_string(err)


def timed_steps(lib, handle, batches, copy_type, steps, warmup, flags, caller="c"):
    """K batch copies between two events on the launch stream; returns (wall s, event ms).
    caller "c": the K calls of smem_bm_copy_batch are issued by a C loop inside the library
    (mf_bm_copy_batch_replay), as a C or C++ program would issue them; "python": one ctypes call
    per batch, which adds about 1 us of interpreter time to every call."""
    stream = lib.mf_xcopy_thread_stream()
    start, stop = lib.mfrt_event_create(), lib.mfrt_event_create()
    call = lib.smem_bm_copy_batch
    nb = len(batches)
    refs = [b.ref for b in batches]
    table = (ctypes.POINTER(native.BatchCopyParams) * nb)(*[ctypes.pointer(b.params) for b in batches])
    for i in range(warmup):
        ret = call(handle, refs[i % nb], copy_type, flags)
        assert ret == 0, native.last_error()
    assert lib.mfrt_stream_sync(stream) == 0
    assert lib.mfrt_device_sync() == 0
    lib.mfrt_event_record(start, stream)
    t0 = time.perf_counter()
    if caller == "c":
        if lib.mf_bm_copy_batch_replay(handle, table, nb, steps, copy_type, flags) != 0:
            raise RuntimeError(native.last_error())
    else:
        for i in range(steps):
            if call(handle, refs[i % nb], copy_type, flags) != 0:
                raise RuntimeError(native.last_error())
    lib.mfrt_event_record(stop, stream)
    # the wait a caller of the API uses; it returns when everything queued on the thread's stream is done
    ret = lib.smem_bm_wait(handle)
    wall = time.perf_counter() - t0
    assert ret == 0, native.last_error()
    assert lib.mfrt_stream_sync(stream) == 0
    assert lib.mfrt_device_sync() == 0
    ms = lib.mfrt_event_elapsed_ms(start, stop)
    lib.mfrt_event_destroy(start)
    lib.mfrt_event_destroy(stop)
    return wall, ms


def threaded_steps(lib, handle, batches, copy_type, steps, threads):
    """The same batches submitted by `threads` host threads started inside the library (no
    interpreter in the loop), each on its own stream as the reference gives every calling thread its
    own; returns the wall-clock seconds from the release of the warmed-up threads to the last wait."""
    nb = len(batches)
    table = (ctypes.POINTER(native.BatchCopyParams) * nb)(*[ctypes.pointer(b.params) for b in batches])
    seconds = ctypes.c_double(0.0)
    if lib.mf_bm_copy_batch_replay_threads(handle, table, nb, steps, copy_type, threads, ctypes.byref(seconds)) != 0:
        raise RuntimeError(native.last_error())
    return seconds.value


def median(values):
    ordered = sorted(values)
    return ordered[len(ordered) // 2]


def steady_state_headline(lib, handle, batches, copy_type, steps, warmup):
    """Ramp, the caller's warm-up steps, then REPETITIONS timed repetitions of `steps` batches.
    Returns (median wall seconds per repetition, median event ms per repetition, all event us per batch)."""
    nb = len(batches)
    table = (ctypes.POINTER(native.BatchCopyParams) * nb)(*[ctypes.pointer(b.params) for b in batches])
    stream = lib.mf_xcopy_thread_stream()
    if lib.mf_bm_copy_batch_replay(handle, table, nb, RAMP_BATCHES + warmup, copy_type, native.ASYNC_COPY_FLAG) != 0:
        raise RuntimeError(native.last_error())
    assert lib.mfrt_stream_sync(stream) == 0
    walls, events = [], []
    for _ in range(REPETITIONS):
        wall, ms = timed_steps(lib, handle, batches, copy_type, steps, 0, native.ASYNC_COPY_FLAG)
        walls.append(wall)
        events.append(ms)
    return median(walls), median(events), sorted(ms * 1e3 / steps for ms in events)


def cpu_baseline(tables, budget_s=12.0):
    """The reference's CPU copy path (single thread, one memcpy per segment, host pool to host
    pool) on the same segment tables: the reference's own DlHybridApi::Memcpy when oracle/_ref was
    built, else the oracle's restatement of it."""
    from tests import oracle_lib
    ref = oracle_lib.reference()
    fn = ref.ref_batch_copy if ref is not None else oracle_lib.oracle().orc_batch_copy_fast
    kind = "reference" if ref is not None else "port"
    pool = POOL_BYTES  # two host pools of 4 GiB, the segment tables used as they are
    block = np.random.default_rng(1).integers(0, 256, 64 * MIB, dtype=np.uint8)
    src_pool = np.empty(pool, dtype=np.uint8)
    dst_pool = np.empty(pool, dtype=np.uint8)
    for i in range(pool // len(block)):
        src_pool[i * len(block):(i + 1) * len(block)] = block
        dst_pool[i * len(block):(i + 1) * len(block)] = 0      # touched before the clock starts
    prepared = []
    for src, dst, lens in tables:
        s = oracle_lib.ptr_array((src_pool.ctypes.data + src).tolist())
        d = oracle_lib.ptr_array((dst_pool.ctypes.data + dst).tolist())
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
        if elapsed > budget_s or batches >= 64 * 400:
            break
    # The same loop on every core the process may use, each thread on its own share of the tables
    # (ctypes releases the GIL during the call): what the host could do at best, for scale.
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, 64))
    totals = [0] * cores

    def worker(t):
        mine = prepared[t::cores] or prepared[:1]
        end = time.perf_counter() + 3.0
        while time.perf_counter() < end:
            for d, s, l, n, payload in mine:
                fn(d, s, l, n)
                totals[t] += payload

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(cores)]
    t1 = time.perf_counter()
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    all_elapsed = time.perf_counter() - t1
    return {
        "value": done_bytes / elapsed / GB,
        "unit": "GB/s",
        "cores": 1,
        "kind": kind,
        "sample": f"{batches} batches of the same 122-segment tables (8994816 B each), 4 GiB host pool to 4 GiB "
                  f"host pool, {elapsed:.1f} s, single thread as the reference runs it; host has {os.cpu_count()} cores",
        "all_cores": {"value": sum(totals) / all_elapsed / GB, "unit": "GB/s", "cores": cores,
                      "sample": f"{cores} threads, each looping over its share of the tables for 3 s "
                                "(destinations of different tables may coincide: bytes are only timed)"},
    }


def kernel_source_digest():
    """Names the kernel sources a counter summary was measured on."""
    import hashlib
    h = hashlib.sha256()
    for name in ("xcopy.hip", "xcopy_plan.h", "window_clock.h"):
        with open(os.path.join(ROOT, "memfabric_hybrid_amd", "csrc", "kernels", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def read_traffic():
    """HBM bytes per launch of the headline kernel, from the committed counter summary (rocprofv3
    --pmc FETCH_SIZE / WRITE_SIZE scaled by the plain copy kernel).  The summary names the kernel
    sources it was measured on; when they have changed since, or the summary is absent, the figure
    is withheld (None) rather than quoted for a kernel it does not describe."""
    path = os.path.join(ROOT, "profiles", "xcopy_inline_kv122_counters.txt")
    traffic, digest = None, None
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch"):
                traffic = float(line.split("=")[1].split()[0])
            if line.startswith("kernel_source_digest"):
                digest = line.split("=")[1].split()[0]
    except OSError:
        return None, "profiles/xcopy_inline_kv122_counters.txt is absent"
    if digest != kernel_source_digest():
        return None, f"counter summary was taken on kernel sources {digest}, these are {kernel_source_digest()}"
    return traffic, "profiles/xcopy_inline_kv122_counters.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy)"


def read_traced_average():
    """Average duration (ns) of the headline kernel under rocprofv3 --kernel-trace, from the committed summary, or None
    where the summary is absent or was taken on other kernel sources.  Under the tracer every dispatch runs alone, with
    its own start-up and write-back: the figure is a kernel duration, not the period of back-to-back launches."""
    path = os.path.join(ROOT, "profiles", "xcopy_inline_kv122_kernel_trace.txt")
    avg, digest = None, None
    try:
        for line in open(path):
            if line.startswith("traced_average_ns"):
                avg = float(line.split("=")[1].split()[0])
            if line.startswith("kernel_source_digest"):
                digest = line.split("=")[1].split()[0]
    except OSError:
        return None
    return avg if digest == kernel_source_digest() else None


def frac(gbps, peak):
    return round(gbps / peak, 4)


def extras_block(lib, pool, dev, batches, tables, steps):
    out = {}
    timer = Timer(lib)
    g2g = int(bm.BmCopyType.G2G)
    payload = batches[0].payload
    handle = pool.handle

    # ---- yardsticks: what this GPU sustains for flat streaming kernels --------------------------------
    half = POOL_BYTES // 2
    yard_lib = native.yardstick()
    sink = lib.mfrt_alloc_device(256)
    yard = {}
    for kind, name, factor in ((0, "copy", 2), (1, "fill", 1), (2, "read", 1)):
        dst = sink if kind == 2 else dev + half
        us, _ = timer.run(lambda k=kind, d=dst: yard_lib.mf_probe_hbm(k, d, dev, 1 << 30, timer.stream), 10)
        yard[name + "_GBps"] = round(factor * (1 << 30) / us / 1e3, 1)
    lib.mfrt_free_device(sink)
    out["hbm_yardstick_1GiB"] = yard
    copy_ceiling = yard["copy_GBps"]

    # ---- KV batch: synchronous calls, concurrency ---------------------------------------------------------
    k = max(500, steps // 4)
    w, _ = timed_steps(lib, handle, batches, g2g, k, 50, 0)
    out["kv122_d2d_sync_call_us"] = round(w * 1e6 / k, 2)
    kp = max(MIN_BATCHES, steps)
    wp, msp = timed_steps(lib, handle, batches, g2g, kp, 100, native.ASYNC_COPY_FLAG, caller="python")
    out["kv122_python_caller"] = {"us_per_batch_wall": round(wp * 1e6 / kp, 2),
                                  "us_per_batch_events": round(msp * 1e3 / kp, 2),
                                  "note": "the headline loop with one ctypes call per batch instead of the C loop"}
    unordered = native.ASYNC_COPY_FLAG | native.MF_COPY_UNORDERED_FLAG
    ku = max(MIN_BATCHES, steps)
    reps_u = sorted(timed_steps(lib, handle, batches, g2g, ku, 0, unordered)[1] * 1e3 / ku for _ in range(5))
    out["kv122_unordered_one_stream"] = {
        "us_per_batch": round(reps_u[2], 2), "hbm_GBps": round(2 * payload / reps_u[2] / 1e3, 1),
        "frac_of_hbm_peak": frac(2 * payload / reps_u[2] / 1e3, HBM_PEAK_GBPS),
        "note": "the headline loop with MF_COPY_UNORDERED_FLAG: the caller declares its batches independent and they are "
                "launched without a barrier, so start-up and drain of consecutive batches overlap; one thread, one stream"}
    # the same with the batches handed to submit threads of the library's (mf_xcopy_unordered_streams): one calling thread,
    # several streams
    fan = {}
    for streams in (3, 4, 6):
        assert lib.mf_xcopy_unordered_streams(streams) == 0
        walls = []
        for _ in range(5):
            w, _ = timed_steps(lib, handle, batches, g2g, ku, 0, unordered)
            walls.append(w * 1e6 / ku)
        fan[f"submit_threads_{streams}"] = {"us_per_batch": round(median(walls), 2), "hbm_GBps": round(2 * payload / median(walls) / 1e3, 1),
                                     "frac_of_hbm_peak": frac(2 * payload / median(walls) / 1e3, HBM_PEAK_GBPS)}
    assert lib.mf_xcopy_unordered_streams(0) == 0
    fan["note"] = (f"{ku} batches with MF_COPY_UNORDERED_FLAG from ONE calling thread, planned by it and launched by submit threads of the "
                   "library's, a stream each; wall clock from the first call to the return of smem_bm_wait (which joins their streams), median of 5")
    out["kv122_unordered_fanout"] = fan
    # the headline loop with the held stores switched off and on in turn, in this process
    held, not_held = [], []
    for _ in range(5):
        assert lib.mf_xcopy_hold_stores(0) == 0
        not_held.append(timed_steps(lib, handle, batches, g2g, ku, 0, native.ASYNC_COPY_FLAG)[1] * 1e3 / ku)
        assert lib.mf_xcopy_hold_stores(-1) == 0
        held.append(timed_steps(lib, handle, batches, g2g, ku, 0, native.ASYNC_COPY_FLAG)[1] * 1e3 / ku)
    out["kv122_held_stores"] = {
        "us_per_batch_not_held": round(median(not_held), 2), "us_per_batch_held": round(median(held), 2),
        "note": "mf_xcopy_hold_stores(0) against the default (every wave of a 960 to 6144 chunk launch keeps its data until the "
                "loads of the whole launch are out, so HBM sees a read burst and then a write burst); 5 alternations, medians"}
    conc = {}
    kc = max(MIN_BATCHES, steps)
    for threads in (1, 2, 4, 8):
        wall = median([threaded_steps(lib, handle, batches, g2g, kc, threads) for _ in range(5)])
        hbm = 2 * payload * kc / wall / GB
        conc[f"threads_{threads}"] = {"us_per_batch": round(wall * 1e6 / kc, 2), "hbm_GBps": round(hbm, 1),
                                      "frac_of_hbm_peak": frac(hbm, HBM_PEAK_GBPS)}
    conc["note"] = (f"{kc} batches shared out over C threads inside the library (mf_bm_copy_batch_replay_threads), each thread "
                    "on its own stream, wall clock from the release of the warmed-up threads to the last wait; median of 5")
    out["kv122_d2d_concurrent_streams"] = conc

    # ---- several requests' KV blocks in one call (the serving case: smem_trans_entry.cpp:363-376 of the reference batches what its
    # caller hands it), and 32 x 1 MiB, the largest block of the reference's own grid that one launch holds in registers
    multi = {}
    eighth = POOL_BYTES // 8
    for requests in (2, 4, 8):
        group = []
        for b in range(16):
            parts = [workloads.kv_batch(0xC1 + 1000 * requests + 8 * b + r, eighth) for r in range(requests)]
            src = np.concatenate([p[0] + np.uint64(r * eighth) for r, p in enumerate(parts)])
            dst = np.concatenate([p[1] + np.uint64(r * eighth) for r, p in enumerate(parts)])
            group.append(Batch(dev + src, dev + dst, np.concatenate([p[2] for p in parts])))
        entry = {}
        for name, hold in (("us_per_call", -1), ("us_per_call_stores_not_held", 0)):
            assert lib.mf_xcopy_hold_stores(hold) == 0
            reps = sorted(timed_steps(lib, handle, group, g2g, 400, 50, native.ASYNC_COPY_FLAG)[1] * 1e3 / 400 for _ in range(5))
            entry[name] = round(reps[2], 2)
        assert lib.mf_xcopy_hold_stores(-1) == 0
        us = entry["us_per_call"]
        entry.update({"segments": group[0].n, "payload_bytes": group[0].payload, "us_per_request": round(us / requests, 2),
                      "hbm_GBps": round(2 * group[0].payload / us / 1e3, 1),
                      "frac_of_hbm_peak": frac(2 * group[0].payload / us / 1e3, HBM_PEAK_GBPS)})
        multi[f"kv_{group[0].n}_segments"] = entry
    blocks = [Batch(dev + np.uint64(b * (64 << 20)) + np.arange(32, dtype=np.uint64) * np.uint64(1 << 20),
                    dev + np.uint64(POOL_BYTES // 2 + b * (64 << 20)) + np.arange(32, dtype=np.uint64)[::-1] * np.uint64(1 << 20),
                    np.full(32, 1 << 20, dtype=np.uint64)) for b in range(16)]
    entry = {}
    for name, hold in (("us_per_call", -1), ("us_per_call_stores_not_held", 0)):
        assert lib.mf_xcopy_hold_stores(hold) == 0
        reps = sorted(timed_steps(lib, handle, blocks, g2g, 400, 50, native.ASYNC_COPY_FLAG)[1] * 1e3 / 400 for _ in range(5))
        entry[name] = round(reps[2], 2)
    assert lib.mf_xcopy_hold_stores(-1) == 0
    entry.update({"payload_bytes": blocks[0].payload, "hbm_GBps": round(2 * blocks[0].payload / entry["us_per_call"] / 1e3, 1),
                  "frac_of_hbm_peak": frac(2 * blocks[0].payload / entry["us_per_call"] / 1e3, HBM_PEAK_GBPS)})
    multi["32_x_1MiB"] = entry
    # ragged tables (no repeating chunk counts: descriptors, prefix and group map are uploaded, the owner of a chunk is looked up)
    for count, lo, hi in ((400, 30000, 70000), (300, 60000, 180000)):
        group = []
        for b in range(16):
            rng = np.random.default_rng(0xE1 + count + b)
            lens = (rng.integers(lo, hi, count) // 128 * 128).astype(np.uint64)
            slot = np.uint64((hi + 4095) // 4096 * 4096)
            src = rng.permutation(2 * count)[:count].astype(np.uint64) * slot
            dst = np.uint64(POOL_BYTES // 2) + rng.permutation(2 * count)[:count].astype(np.uint64) * slot
            group.append(Batch(dev + src, dev + dst, lens))
        entry = {}
        for name, hold in (("us_per_call", -1), ("us_per_call_stores_not_held", 0)):
            assert lib.mf_xcopy_hold_stores(hold) == 0
            reps = sorted(timed_steps(lib, handle, group, g2g, 300, 30, native.ASYNC_COPY_FLAG)[1] * 1e3 / 300 for _ in range(5))
            entry[name] = round(reps[2], 2)
        assert lib.mf_xcopy_hold_stores(-1) == 0
        entry.update({"segments": count, "payload_bytes": group[0].payload,
                      "hbm_GBps": round(2 * group[0].payload / entry["us_per_call"] / 1e3, 1),
                      "frac_of_hbm_peak": frac(2 * group[0].payload / entry["us_per_call"] / 1e3, HBM_PEAK_GBPS)})
        multi[f"ragged_{count}_segments_{lo // 1000}_to_{hi // 1000}_KB"] = entry
    multi["note"] = ("asynchronous smem_bm_copy_batch calls back to back on one stream, 16 tables in turn, HIP events, median of 5 runs; more than "
                     "128 segments take the table form (descriptors read from the pinned staging slot), up to 24 MiB in 4 KiB chunks and up "
                     "to 64 MiB in 16 KiB chunks with the stores held back until the loads of the launch are out")
    out["batches_of_several_requests"] = multi

    # ---- the grid the reference publishes for its transfer benchmark (example/trans/perf/README.md:61-70 there:
    # 32 equal blocks per batch, blocking calls, GB/s = block * 32 / time per call), here HBM to HBM on one GPU
    grid = []
    for block in (32 << 10, 64 << 10, 128 << 10, 256 << 10, 512 << 10, 1 << 20, 2 << 20, 4 << 20, 8 << 20, 16 << 20):
        src_off = np.arange(32, dtype=np.uint64) * block
        dst_off = (POOL_BYTES // 2) + np.arange(32, dtype=np.uint64) * block
        b = Batch(dev + src_off, dev + dst_off, np.full(32, block, dtype=np.uint64))
        for _ in range(20):     # the first calls after a different workload take 2 us longer
            lib.smem_bm_copy_batch(handle, b.ref, g2g, 0)
        t0 = time.perf_counter()
        for _ in range(100):
            lib.smem_bm_copy_batch(handle, b.ref, g2g, 0)
        per_call = (time.perf_counter() - t0) / 100
        grid.append({"block_KiB": block >> 10, "us_per_call": round(per_call * 1e6, 1),
                     "payload_GBps": round(32 * block / per_call / GB, 1)})
    out["batch32_blocking_calls_d2d"] = grid

    # ---- KV batch over the host link ------------------------------------------------------------------------
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    split = [workloads.kv_batch(0xD1 + b, POOL_BYTES, same_pool=False) for b in range(16)]
    for name, bs in (("kv122_h2d", [Batch(host + s, dev + d, l) for s, d, l in split]),
                     ("kv122_d2h", [Batch(dev + s, host + d, l) for s, d, l in split])):
        kk = max(100, steps // 20)
        _, ms = timed_steps(lib, handle, bs, g2g, kk, 10, native.ASYNC_COPY_FLAG)
        gbps = payload * kk / (ms * 1e-3) / GB
        out[name] = {"GBps": round(gbps, 2), "frac_of_link_peak": frac(gbps, LINK_PEAK_GBPS),
                     "us_per_batch": round(ms * 1e3 / kk, 1)}
    for name, (d, s) in (("dma_h2d_1GiB", (dev, host)), ("dma_d2h_1GiB", (host, dev))):
        us, _ = timer.run(lambda d=d, s=s: lib.mfrt_memcpy_async(d, s, 1 << 30, timer.stream), 3, warm=1)
        out[name + "_GBps"] = round((1 << 30) / us / 1e3, 2)   # the runtime's DMA engines, for comparison

    # ---- pageable caller memory: CPU memcpy into a pinned ring overlapped with the launches (PCIe- and memcpy-inclusive)
    page_host = np.empty(1 << 30, dtype=np.uint8)
    page_host[:] = 7
    php = page_host.ctypes.data
    pageable = {}
    for name, ct, params in (("h2d_1GiB", int(bm.BmCopyType.H2G), native.SmemCopyParams(php, dev, 1 << 30)),
                             ("d2h_1GiB", int(bm.BmCopyType.G2H), native.SmemCopyParams(dev, php, 1 << 30))):
        lib.smem_bm_copy(handle, ctypes.byref(params), ct, 0)
        t0 = time.perf_counter()
        for _ in range(2):
            if lib.smem_bm_copy(handle, ctypes.byref(params), ct, 0) != 0:
                raise RuntimeError(native.last_error())
        pageable[name + "_GBps"] = round(2 * (1 << 30) / (time.perf_counter() - t0) / 1e9, 2)
    t0 = time.perf_counter()
    ctypes.memmove(php, php + (1 << 29), 1 << 29)
    pageable["host_memmove_GBps"] = round((1 << 29) / (time.perf_counter() - t0) / 1e9, 2)
    out["pageable_host_memory"] = pageable
    del page_host

    # ---- large single copies through smem_bm_copy --------------------------------------------------------------
    big = {}
    for size_name, nbytes in (("1GiB", 1 << 30), ("2GiB", 2 << 30)):
        for dname, (s, d, peak, factor) in (("d2d", (dev, dev + half, HBM_PEAK_GBPS, 2)),
                                            ("h2d", (host, dev, LINK_PEAK_GBPS, 1)),
                                            ("d2h", (dev, host, LINK_PEAK_GBPS, 1))):
            params = native.SmemCopyParams(s, d, nbytes)
            us, _ = timer.run(lambda p=params: lib.smem_bm_copy(handle, ctypes.byref(p), g2g, native.ASYNC_COPY_FLAG),
                              10 if dname == "d2d" else 2, warm=1)
            gbps = factor * nbytes / us / 1e3
            big[f"{dname}_{size_name}"] = {"GBps": round(gbps, 1), "frac_of_peak": frac(gbps, peak), "us": round(us, 1)}
    out["single_copy"] = big
    return out, copy_ceiling


def extras_transfer(lib, dev, batches, steps):
    """The same KV batches through the transfer front-end: a Prefill object writes into the pool
    a Decode object registered, submitted on one stream (smem_trans_batch_write_submit)."""
    from memfabric_hybrid_amd.transfer import TransferEngine
    prefill, decode = TransferEngine(), TransferEngine()
    if prefill.initialize("tcp://127.0.0.1:15432", "127.0.0.1:15321", "Prefill", 0) != 0 or \
            decode.initialize("tcp://127.0.0.1:15432", "127.0.0.1:15322", "Decode", 0) != 0 or \
            decode.register_memory(dev, POOL_BYTES) != 0:
        return {"error": native.last_error()}
    timer = Timer(lib)
    peer = b"127.0.0.1:15322"
    call, handle, stream = lib.smem_trans_batch_write_submit, prefill._handle, timer.stream
    i = [0]

    def step():
        b = batches[i[0] % len(batches)]
        i[0] += 1
        if call(handle, b.srcs, peer, b.dsts, b.lens, b.n, stream, 0) != 0:
            raise RuntimeError(native.last_error())

    k = max(400, steps // 4)
    py_us, py_wall_us = timer.run(step, k, warm=50)
    # the same calls issued by a C loop inside the library, as for the headline
    nb = len(batches)
    table = (ctypes.POINTER(native.BatchCopyParams) * nb)(*[ctypes.pointer(b.params) for b in batches])
    kc = max(MIN_BATCHES, steps)

    def replay():
        if lib.mf_trans_batch_write_replay(handle, table, nb, kc, peer, stream) != 0:
            raise RuntimeError(native.last_error())

    reps = sorted(timer.run(replay, 1, warm=1)[0] / kc for _ in range(5))
    us = reps[2]
    hbm = 2 * batches[0].payload / us / 1e3
    decode.unregister_memory(dev)
    prefill.destroy()
    decode.destroy()
    prefill.unInitialize()
    return {"api": "smem_trans_batch_write_submit, Prefill -> Decode object in one process, one stream",
            "us_per_batch": round(us, 2), "hbm_GBps": round(hbm, 1), "frac_of_hbm_peak": frac(hbm, HBM_PEAK_GBPS),
            "python_caller_us_per_batch": round(py_us, 2), "python_caller_wall_us_per_batch": round(py_wall_us, 2),
            "note": "us_per_batch: the calls issued by a C loop (mf_trans_batch_write_replay), median of 5 runs; python_caller: one ctypes call per batch"}


def extras_plugin(lib, dev, tables, steps):
    """The same KV batches through the two-symbol plugin, as the reference's SDMA operator drives it:
    a pinned parameter table per call, a completion word, 32 as the word's value."""
    plug = native.plugin()
    slot = 16384 * 24
    params = lib.mfrt_alloc_host(len(tables) * slot + 4096)
    if not params:
        return {"error": "allocation failed"}
    for b, (s, d, l) in enumerate(tables):
        t = np.ctypeslib.as_array((ctypes.c_uint64 * (3 * len(l))).from_address(params + b * slot))
        t[0::3], t[1::3], t[2::3] = dev + s, dev + d, l
    mask = params + len(tables) * slot
    timer = Timer(lib)
    i = [0]

    def step():
        plug.hybm_batch_copy_extend(params + (i[0] % len(tables)) * slot, len(tables[0][2]), mask, 32, timer.stream)
        i[0] += 1

    us, _ = timer.run(step, max(400, steps // 4), warm=50)
    hbm = 2 * int(tables[0][2].sum()) / us / 1e3
    ok = ctypes.c_uint64.from_address(mask).value == 32
    lib.mfrt_free_host(params)
    return {"api": "hybm_batch_copy_extend(pinned table, 122, mask, 32, stream)", "us_per_batch": round(us, 2),
            "hbm_GBps": round(hbm, 1), "frac_of_hbm_peak": frac(hbm, HBM_PEAK_GBPS), "mask_ok": ok}


def extras_paged(lib):
    """Paged KV gather/scatter: 4096 distinct 32 KiB pages out of a 40 GiB pool."""
    page, count = 32768, 4096
    pool_bytes = 40 << 30
    pool = lib.mfrt_alloc_device(pool_bytes)
    buf = lib.mfrt_alloc_device(count * page * 4)
    if not pool or not buf:
        return {"error": "allocation failed"}
    timer = Timer(lib)
    sets = []
    for b in range(4):
        ids = workloads.page_ids(0xC3 + b, pool_bytes // page, count)
        flat = buf + b * count * page + np.arange(count, dtype=np.uint64) * page
        sets.append((native.u64_array((pool + ids * page).tolist()), native.u64_array(flat.tolist()),
                     native.u64_array([page] * count)))
    i = [0]

    def gather():
        s, d, l = sets[i[0] % 4]
        i[0] += 1
        assert lib.mf_xcopy_batch(s, d, l, count, native.ROUTE_HBM, None) == 0

    def scatter():
        s, d, l = sets[i[0] % 4]
        i[0] += 1
        assert lib.mf_xcopy_batch(d, s, l, count, native.ROUTE_HBM, None) == 0

    res = {}
    for name, fn in (("gather", gather), ("scatter", scatter)):
        us, _ = timer.run(fn, 40, warm=10)   # the warm-up sizes all staging slots of the thread
        hbm = 2 * count * page / us / 1e3
        res[name] = {"us": round(us, 1), "hbm_GBps": round(hbm, 1), "frac_of_hbm_peak": frac(hbm, HBM_PEAK_GBPS)}
    res["shape"] = "4096 x 32 KiB pages, 40 GiB pool, one K-or-V plane of one layer per call (134 217 728 B)"
    lib.mfrt_device_sync()

    def device_table(src, dst, lens):
        t = np.stack([np.asarray(src, dtype=np.uint64), np.asarray(dst, dtype=np.uint64), np.asarray(lens, dtype=np.uint64)], axis=1)
        t = np.ascontiguousarray(t).reshape(-1)
        p = lib.mfrt_alloc_device(t.nbytes)
        assert p and lib.mfrt_memcpy(p, t.ctypes.data, t.nbytes) == 0
        return p

    # the same gather with its {src, dst, len} table resident in device memory (the plugin ABI's other legal form): planned on the GPU
    ids = workloads.page_ids(0xC3, pool_bytes // page, count)
    tab = device_table(pool + ids * page, buf + np.arange(count, dtype=np.uint64) * page, np.full(count, page))
    us, _ = timer.run(lambda: lib.mf_xcopy_device_table(tab, count, native.ROUTE_HBM, None), 40, warm=10)
    table_path = {"device_table_4096_pages": {"us": round(us, 1), "hbm_GBps": round(2 * count * page / us / 1e3, 1),
                                               "frac_of_hbm_peak": frac(2 * count * page / us / 1e3, HBM_PEAK_GBPS),
                                               "us_descriptors_from_host_arrays": res["gather"]["us"]}}
    lib.mfrt_device_sync()
    lib.mfrt_free_device(tab)
    lib.mfrt_free_device(buf)
    # 16 384 ragged segments of 2 to 262 KB at odd addresses: no pattern, the group map finds a chunk's segment
    rng = np.random.default_rng(7)
    n_ragged, slot = 16384, 512 << 10
    lens = rng.integers(2000, 262144, size=n_ragged).astype(np.uint64)
    src = pool + rng.permutation(2 * n_ragged)[:n_ragged].astype(np.uint64) * np.uint64(slot) + rng.integers(0, 64, n_ragged).astype(np.uint64)
    dst = pool + np.uint64(20 << 30) + np.arange(n_ragged, dtype=np.uint64) * np.uint64(slot) + rng.integers(0, 64, n_ragged).astype(np.uint64)
    s_r, d_r, l_r = native.u64_array(src.tolist()), native.u64_array(dst.tolist()), native.u64_array(lens.tolist())
    moved = int(lens.sum())
    us, _ = timer.run(lambda: lib.mf_xcopy_batch(s_r, d_r, l_r, n_ragged, native.ROUTE_HBM, None), 20, warm=10)
    tab = device_table(src, dst, lens)
    us_dev, _ = timer.run(lambda: lib.mf_xcopy_device_table(tab, n_ragged, native.ROUTE_HBM, None), 20, warm=10)
    table_path["ragged_16384"] = {"payload_bytes": moved, "us": round(us, 1), "hbm_GBps": round(2 * moved / us / 1e3, 1),
                                  "frac_of_hbm_peak": frac(2 * moved / us / 1e3, HBM_PEAK_GBPS),
                                  "us_table_in_device_memory": round(us_dev, 1),
                                  "frac_of_hbm_peak_table_in_device_memory": frac(2 * moved / us_dev / 1e3, HBM_PEAK_GBPS)}
    lib.mfrt_device_sync()
    lib.mfrt_free_device(tab)
    # The whole set of a 32-layer model (K and V planes: 64 x 4096 pages) as ONE call of 262 144 descriptors.
    planes = 64
    big = lib.mfrt_alloc_device(planes * count * page)
    if big:
        ids = np.concatenate([workloads.page_ids(0xC3 + 16 + b, pool_bytes // page, count) for b in range(planes)])
        total = planes * count
        s_all = native.u64_array((pool + ids * page).tolist())
        d_all = native.u64_array((big + np.arange(total, dtype=np.uint64) * page).tolist())
        l_all = native.u64_array([page] * total)

        def gather_all():
            assert lib.mf_xcopy_batch(s_all, d_all, l_all, total, native.ROUTE_HBM, None) == 0

        us, _ = timer.run(gather_all, 8, warm=9)   # the warm-up sizes all descriptor staging slots
        hbm = 2 * total * page / us / 1e3
        res["gather_full_set_one_call"] = {"descriptors": total, "us": round(us, 1), "hbm_GBps": round(hbm, 1),
                                           "frac_of_hbm_peak": frac(hbm, HBM_PEAK_GBPS)}
        tab = device_table(pool + ids * page, big + np.arange(total, dtype=np.uint64) * page, np.full(total, page))
        us_dev, _ = timer.run(lambda: lib.mf_xcopy_device_table(tab, total, native.ROUTE_HBM, None), 8, warm=4)
        table_path["device_table_262144_pages"] = {"us": round(us_dev, 1), "hbm_GBps": round(2 * total * page / us_dev / 1e3, 1),
                                                   "frac_of_hbm_peak": frac(2 * total * page / us_dev / 1e3, HBM_PEAK_GBPS),
                                                   "us_descriptors_from_host_arrays": round(us, 1)}
        lib.mfrt_device_sync()
        lib.mfrt_free_device(tab)
        lib.mfrt_free_device(big)
    table_path["note"] = ("device_table_*: mf_xcopy_device_table, the table planned on the GPU (chunk prefix, group map, and the repeating chunk "
                          "counts of equal pages found there) in one launch up to 8192 segments, two beyond, in front of the copy launch; "
                          "ragged_16384: mf_xcopy_batch from host arrays (descriptors, prefix and group map uploaded by a launch of its own) "
                          "and the same table resident in device memory")
    res["table_path"] = table_path
    lib.mfrt_free_device(pool)
    return res


MOE_SHAPE = (8192, 7168, 8, 256)   # tokens, hidden, top-k, experts


def extras_moe(lib):
    T, H, K, E = MOE_SHAPE
    x, logits = workloads.moe_inputs(0xC4, T, H, E, K)
    topk, w = workloads.moe_route(logits, K)

    def dev_of(a):
        p = lib.mfrt_alloc_device(a.nbytes)
        assert lib.mfrt_memcpy(p, a.ctypes.data, a.nbytes) == 0
        return p

    dx, dt, dw = dev_of(x), dev_of(topk), dev_of(w)
    out = lib.mfrt_alloc_device(T * K * H * 2)
    y = lib.mfrt_alloc_device(T * H * 2)
    counts, offs = lib.mfrt_alloc_device(E * 4), lib.mfrt_alloc_device(E * 4)
    row, src = lib.mfrt_alloc_device(T * K * 4), lib.mfrt_alloc_device(T * K * 4)
    wsb = lib.mf_moe_workspace_bytes(T, K, E)
    ws = lib.mfrt_alloc_device(wsb)
    timer = Timer(lib)

    def dispatch():
        assert lib.mf_moe_dispatch(dx, dt, T, H, K, E, out, counts, offs, row, src, ws, wsb, None) == 0

    def combine():
        assert lib.mf_moe_combine(out, row, dw, T, H, K, y, None) == 0

    d_us, _ = timer.run(dispatch, 30, warm=3)
    # the combine as shipped (waves that stay and alternate between reading and writing) and, on the same box in
    # turn, the form with one workgroup per slice that it replaces at this size
    shipped, one_shot = [], []
    for _ in range(3):
        shipped.append(timer.run(combine, 30, warm=3)[0])
        assert lib.mf_moe_combine_windows(0, 0) == 0
        one_shot.append(timer.run(combine, 30, warm=3)[0])
        assert lib.mf_moe_combine_windows(*native.MOE_COMBINE_WINDOWS_DEFAULT) == 0
    c_us = sorted(shipped)[1]
    d_bytes = T * H * 2 + T * K * H * 2 + T * K * 4
    c_bytes = T * K * H * 2 + T * K * 4 + T * K * 4 + T * H * 2
    res = {
        "shape": "8192 tokens x 7168 bf16, 256 experts, top-8 (local share)",
        "dispatch": {"us": round(d_us, 1), "algorithmic_bytes": d_bytes, "hbm_GBps": round(d_bytes / d_us / 1e3, 1),
                     "frac_of_hbm_peak": frac(d_bytes / d_us / 1e3, HBM_PEAK_GBPS)},
        "combine": {"us": round(c_us, 1), "algorithmic_bytes": c_bytes, "hbm_GBps": round(c_bytes / c_us / 1e3, 1),
                    "frac_of_hbm_peak": frac(c_bytes / c_us / 1e3, HBM_PEAK_GBPS)},
    }
    res["combine"]["us_one_workgroup_per_slice"] = round(sorted(one_shot)[1], 1)
    both = (d_bytes + c_bytes) / (d_us + c_us) / 1e3
    res["dispatch_plus_combine"] = {"hbm_GBps": round(both, 1), "frac_of_hbm_peak": frac(both, HBM_PEAK_GBPS)}
    lib.mfrt_device_sync()
    for p in (dx, dt, dw, out, y, counts, offs, row, src, ws):
        lib.mfrt_free_device(p)
    return res


def cpu_baseline_moe():
    """The MoE workload on one host core: the oracle's dispatch (stable counting sort + row copies)
    and combine (fp32 FMA chain, one rounding to bf16), one pass each at full size."""
    from tests import oracle_lib
    oracle = oracle_lib.oracle()
    T, H, K, E = MOE_SHAPE
    x, logits = workloads.moe_inputs(0xC4, T, H, E, K)
    topk, w = workloads.moe_route(logits, K)
    out = np.zeros((T * K, H), dtype=np.uint16)
    counts, offsets = np.zeros(E, dtype=np.int32), np.zeros(E, dtype=np.int32)
    row_of, src_of = np.zeros(T * K, dtype=np.int32), np.zeros(T * K, dtype=np.int32)
    y = np.zeros((T, H), dtype=np.uint16)
    t0 = time.perf_counter()
    ret = oracle.orc_moe_dispatch(x.ctypes.data, topk.ctypes.data, T, H, K, E, out.ctypes.data, counts.ctypes.data,
                                  offsets.ctypes.data, row_of.ctypes.data, src_of.ctypes.data)
    t1 = time.perf_counter()
    assert ret == 0
    oracle.orc_moe_combine(out.ctypes.data, row_of.ctypes.data, w.ctypes.data, T, H, K, y.ctypes.data)
    t2 = time.perf_counter()
    d_bytes = T * H * 2 + T * K * H * 2 + T * K * 4
    c_bytes = T * K * H * 2 + T * K * 4 + T * K * 4 + T * H * 2
    # the combine once more with the tokens shared out over all host cores (tokens are independent)
    cores = min(16, os.cpu_count() or 1)
    bounds = [T * i // cores for i in range(cores + 1)]

    def part(i):
        a, b = bounds[i], bounds[i + 1]
        oracle.orc_moe_combine(out.ctypes.data, row_of.ctypes.data + a * K * 4, w.ctypes.data + a * K * 4, b - a, H, K,
                               y.ctypes.data + a * H * 2)

    workers = [threading.Thread(target=part, args=(i,)) for i in range(cores)]
    t3 = time.perf_counter()
    for t in workers:
        t.start()
    for t in workers:
        t.join()
    t4 = time.perf_counter()
    return {"cores": 1, "kind": "port", "sample": "one pass each at the full shape",
            "dispatch": {"ms": round((t1 - t0) * 1e3, 1), "GBps": round(d_bytes / (t1 - t0) / GB, 2)},
            "combine": {"ms": round((t2 - t1) * 1e3, 1), "GBps": round(c_bytes / (t2 - t1) / GB, 2)},
            "combine_all_cores": {"cores": cores, "ms": round((t4 - t3) * 1e3, 1), "GBps": round(c_bytes / (t4 - t3) / GB, 2)}}


def extras_reshard(lib):
    tensors = workloads.reshard_tensors()
    layers = workloads.RESHARD_LAYERS
    _, _, s_bytes, d_bytes = workloads.reshard_layout(tensors, layers)
    sp, dp = lib.mfrt_alloc_device(s_bytes), lib.mfrt_alloc_device(d_bytes)
    if not sp or not dp:
        return {"error": "allocation failed"}
    lib.mfrt_memset(sp, 0x5A, s_bytes)   # weights that were written at some point, as a checkpoint in HBM is
    segments, rects = workloads.reshard_plan(tensors, layers, sp, dp)
    s_arr = native.u64_array([s for s, _, _ in segments])
    d_arr = native.u64_array([d for _, d, _ in segments])
    l_arr = native.u64_array([n for _, _, n in segments])
    descs = (native.Copy2dDesc * len(rects))()
    for i, r in enumerate(rects):
        descs[i] = native.Copy2dDesc(*[int(v) for v in r])
    timer = Timer(lib)

    def run():
        assert lib.mf_xcopy_batch(s_arr, d_arr, l_arr, len(segments), native.ROUTE_HBM, None) == 0
        assert lib.mf_xcopy_2d_batch(descs, len(rects), native.ROUTE_HBM, None) == 0

    us, _ = timer.run(run, 5, warm=8)   # the warm-up sizes all staging slots of the thread
    moved = sum(n for _, _, n in segments) + sum(r[2] * r[3] for r in rects)
    hbm = 2 * moved / us / 1e3
    lib.mfrt_device_sync()
    lib.mfrt_free_device(sp)
    lib.mfrt_free_device(dp)
    return {"shape": "28 layers, hidden 3584, FFN 18944, 28 Q / 4 KV heads, TP8 storage -> TP4 layout",
            "bytes_moved": moved, "source_bytes": s_bytes, "segments": len(segments), "rectangles": len(rects),
            "us": round(us, 1), "hbm_GBps": round(hbm, 1), "frac_of_hbm_peak": frac(hbm, HBM_PEAK_GBPS)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=400)
    ap.add_argument("--no-extras", action="store_true", help="headline only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--calibrate", action="store_true", help="only run the plain copy kernel (counter calibration)")
    ap.add_argument("--fitted-rules", action="store_true",
                    help="hybm_init keeps the fitted hold and window rules instead of timing them on this GPU (MF_HIP_CALIBRATE=0): for "
                         "runs under a tracer, which serialises dispatches and would make the check switch the held stores off")
    ap.add_argument("--phases", action="store_true",
                    help="only run the stand-alone program that takes KV batches apart (bench_phases/mf_batch_phases) and print its JSON")
    ap.add_argument("--only", choices=("paged", "reshard", "moe"),
                    help="run one of the larger workloads alone and print its JSON (what the counter summaries under profiles/ are taken on)")
    ap.add_argument("phase_args", nargs="*", help="with --phases: requests per batch to take apart (1 2 4 8), default 1 and 4")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is a single-GPU data plane (no collectives, no sharding); run with --gpus 1")

    if args.fitted_rules:
        os.environ["MF_HIP_CALIBRATE"] = "0"

    if args.phases:
        # a child process of its own, started before this one touches the GPU
        import subprocess
        exe = os.path.join(ROOT, "bench_phases", "mf_batch_phases")
        # not part of the product build: compiled on demand, and again whenever the kernel sources it includes have changed
        subprocess.run(["make", "-C", os.path.join(ROOT, "bench_phases")], check=True, stdout=subprocess.DEVNULL)
        done = subprocess.run([exe] + args.phase_args, stdout=subprocess.PIPE, text=True, timeout=600)
        sys.stdout.write(done.stdout)
        sys.exit(done.returncode)

    lib = native.lib()
    if args.calibrate:
        # counter calibration load: five launches of the plain copy kernel, 1 GiB read + 1 GiB written each
        assert lib.hybm_init(0, 0) == 0, native.last_error()
        a, b = lib.mfrt_alloc_device(1 << 30), lib.mfrt_alloc_device(1 << 30)
        for _ in range(5):
            assert native.yardstick().mf_probe_hbm(0, b, a, 1 << 30, None) == 0
        assert lib.mfrt_device_sync() == 0
        print(json.dumps({"calibrate": "ProbeCopyKernel", "launches": 5, "bytes_read_per_launch": 1 << 30,
                          "bytes_written_per_launch": 1 << 30}))
        lib.hybm_uninit()
        return
    if args.only:
        assert lib.hybm_init(0, 0) == 0, native.last_error()
        fn = {"paged": extras_paged, "reshard": extras_reshard, "moe": extras_moe}[args.only]
        print(json.dumps({args.only: fn(lib)}))
        lib.hybm_uninit()
        return
    assert bm.initialize("tcp://127.0.0.1:0", 1, 0) == 0, native.last_error()
    want_host = 0 if args.no_extras else POOL_BYTES
    pool = bm.create(0, want_host, POOL_BYTES)
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    fill_device_pool(lib, dev, POOL_BYTES, 0xC1)

    tables = [workloads.kv_batch(0xC1 + b, POOL_BYTES) for b in range(TABLES)]
    batches = [Batch(dev + s, dev + d, l) for s, d, l in tables]
    payload = batches[0].payload
    g2g = int(bm.BmCopyType.G2G)

    # The submitting thread runs where a launch costs it least (mf_pin_thread_near_gpu: 3.1 against 4.3 us per call
    # between the two halves of the CPUs on the hosts of this pool, which decides whether the host or the GPU sets
    # the pace of this loop); extras.kv122_any_cpu has the same loop with the scheduler free to put it anywhere.
    all_cpus = sorted(os.sched_getaffinity(0))
    cpu_ids, cpu_us = (ctypes.c_uint32 * 1024)(), (ctypes.c_float * 1024)()
    measured = lib.mf_host_launch_costs(cpu_ids, cpu_us, 1024)
    launch_us_by_cpu = {int(cpu_ids[i]): round(float(cpu_us[i]), 2) for i in range(max(measured, 0))}
    kept = lib.mf_pin_thread_near_gpu()
    near_cpus = sorted(os.sched_getaffinity(0))

    cal_on, cal_delta, cal_rate, cal_aligned = ctypes.c_int32(0), ctypes.c_int32(0), ctypes.c_uint32(0), ctypes.c_uint32(0)
    cal_long = ctypes.c_uint32(0)
    cal_us = (ctypes.c_float * 8)()
    cal_ran = lib.mf_xcopy_calibration(ctypes.byref(cal_on), ctypes.byref(cal_delta), ctypes.byref(cal_rate), ctypes.byref(cal_aligned), ctypes.byref(cal_long), cal_us)
    calibration = {"ran": bool(cal_ran), "held_stores": bool(cal_on.value), "hold_delta_ns": cal_delta.value,
                   "window_MBps": cal_rate.value, "window_MBps_aligned_segments": cal_aligned.value, "window_MBps_long_aligned_segments": cal_long.value,
                   "us_per_2196_chunk_batch_not_held_and_held_rule_minus_200_rule_plus_200": [round(v, 2) for v in cal_us[:4]],
                   "us_per_512MiB_copy_plain_windows_default_windows_94_percent_windows_long_segment_rate": [round(v, 1) for v in cal_us[4:]],
                   "note": "measured by hybm_init on this GPU (about 15 ms): the wait of the held stores is the fitted rule plus the offset "
                           "that was fastest here, the window rate the faster of two (higher rates for segments on cache lines where a long one "
                           "held it), either form off where it does not gain"}

    deck = (ctypes.c_uint32 * 16)()
    stream_queues = {"hardware_queue_of_each_stream_in_hand_out_order": list(deck[:min(16, lib.mf_xcopy_stream_queues(deck, 16))]),
                     "note": "hybm_init asks the GPU which of its first streams share a hardware queue (launches on such streams run one "
                             "after the other) and hands out one stream of every queue before the second of any: the calling thread holds "
                             "the first, threads and submit threads that come later the next ones"}
    wall, ms, rep_us = steady_state_headline(lib, pool.handle, batches, g2g, args.steps, args.warmup)
    per_launch_us = ms * 1e3 / args.steps
    value = payload * args.steps / wall / GB
    achieved = 2 * payload / (per_launch_us * 1e-6) / GB
    traffic, traffic_source = read_traffic()
    traced_ns = read_traced_average()

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
            "api": "smem_bm_copy_batch(SMEMB_COPY_G2G, ASYNC_COPY_FLAG) on one stream + one wait; the K calls are "
                   "issued by a C loop (mf_bm_copy_batch_replay), extras.kv122_python_caller has one ctypes call per batch",
            "timing": f"submitting thread pinned near the GPU; untimed ramp of {RAMP_BATCHES} batches + --warmup, then {REPETITIONS} repetitions of --steps batches, "
                      "each between two synchronisations; ms_per_step / value: median repetition by the host clock, "
                      "from the first call to the return of smem_bm_wait (behind a queue of up to 256 MiB it polls a word that a "
                      "one-lane launch stores behind the last batch, behind more it is hipStreamSynchronize; hipStreamSynchronize "
                      "and hipDeviceSynchronize follow before the next repetition), roofline: median repetition by HIP events",
            "payload_bytes": payload,
            "cu_count": lib.mfrt_cu_count(),
            "calibration": calibration,
            "stream_queues": stream_queues,
            "submitting_thread": {"empty_launch_us_by_cpu": launch_us_by_cpu, "runs_on_cpus": near_cpus if kept > 0 else all_cpus,
                                  "note": "mf_pin_thread_near_gpu: the CPUs from which a launch with a full argument block is "
                                          "cheapest, measured at start; the threads of the concurrency extras inherit the set"},
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "frac_traced": None if traced_ns is None else round(2 * payload / traced_ns / HBM_PEAK_GBPS, 4),
            "frac_traced_note": "algorithmic bytes / the kernel's average duration under rocprofv3 --kernel-trace "
                                "(profiles/xcopy_inline_kv122_kernel_trace.txt): there every dispatch runs alone, so this is "
                                "a kernel duration, longer than the period of back-to-back launches that frac is computed from",
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel": "XcopyInlineKernel<true, 1, 1> (one launch per batch; stores held back until the loads of the launch are out)",
            "algorithmic_bytes_per_launch": 2 * payload,
            "avg_launch_us": per_launch_us,
            "repetitions_us_per_launch": {"n": len(rep_us), "min": round(rep_us[0], 3), "median": round(rep_us[len(rep_us) // 2], 3),
                                          "max": round(rep_us[-1], 3)},
        },
    }

    def guarded(fn, *fargs):
        """The other workloads must not cost the headline line: a failure is recorded, not raised."""
        try:
            return fn(*fargs)
        except Exception as exc:  # noqa: BLE001
            return {"error": repr(exc)[:300]}

    extras = {}
    if not args.no_extras:
        def any_cpu():
            os.sched_setaffinity(0, all_cpus)
            try:
                w, m, _ = steady_state_headline(lib, pool.handle, batches, g2g, max(args.steps, 2000), 0)
                n = max(args.steps, 2000)
                return {"us_per_batch_wall": round(w * 1e6 / n, 2), "us_per_batch_events": round(m * 1e3 / n, 2),
                        "note": "the headline loop without the pinning: the scheduler may run the submitting thread on any of "
                                "the process's CPUs"}
            finally:
                os.sched_setaffinity(0, near_cpus)
        any_cpu_result = guarded(any_cpu)
        block = guarded(extras_block, lib, pool, dev, batches, tables, args.steps)
        if isinstance(block, tuple):
            extras, copy_ceiling = block
            result["roofline"]["frac_of_measured_copy_ceiling"] = frac(achieved, copy_ceiling)
        else:
            extras = {"kv122_and_link": block}
        extras["kv122_any_cpu"] = any_cpu_result
        extras["kv122_transfer_write"] = guarded(extras_transfer, lib, dev, batches, args.steps)
        extras["kv122_plugin"] = guarded(extras_plugin, lib, dev, tables, args.steps)
    pool.destroy()  # give the pools back before the larger workloads allocate
    if not args.no_extras:
        # in order of growing footprint: buffers allocated after the 40 GiB pool has been freed again land on
        # memory that every kernel streams about 3 % slower from (MoE combine 181.7 instead of 177 us)
        extras["moe_local"] = guarded(extras_moe, lib)
        extras["reshard_tp8_to_tp4"] = guarded(extras_reshard, lib)
        extras["paged_kv_40GiB"] = guarded(extras_paged, lib)
        result["extras"] = extras

    os.sched_setaffinity(0, all_cpus)   # the CPU baselines use every core
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(tables)
        if not args.no_extras:
            result["cpu_baseline"]["moe_local"] = guarded(cpu_baseline_moe)

    bm.uninitialize()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
