#!/usr/bin/env python3
"""Benchmark of the gather + scatter hot path on one MI355X.

One step = one pass of the hot path (descriptor build, gather, descriptor
build, scatter + header rewrite) over one call's worth of synthetic input that
is already resident in HBM.  The default workload is the ResNet-50-sized one:
16 requests x 602112 B in 431 frames of <= 1400 B, 2048-byte slots, frames
permuted inside a request; `--batches-per-launch B` lays B such batches side by
side in the ring so that one call moves B batches (B = 1 is the single-batch
call).  Ring copies are rotated between steps so that reads come from HBM and
not from the 256 MB memory-side cache.

Prints ONE JSON line: whole-job GB/s over the algorithmic bytes
(2*payload + 16*frames gather, 2*payload + 2*58*frames scatter), the roofline
of the dominant kernel from HIP-event kernel times, requests/s of all five
workloads and the CPU oracle timed on this host as a baseline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes the copy kernels of one call move, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this file (--calib-copy --steps 40 --warmup 5), each counter scaled by what it reads for a plain
# 512 MiB device copy in the same run (FETCH_SIZE x 2.000 KiB, WRITE_SIZE x 1.000 KiB).  Keyed by
# (workload, batches per launch, kernel family); the default call: 340.5 MB read + 313.1 MB written.
# bert's scatter is both of its kernels (full frames + short remainder frames), jumbo's the copy
# phase without the 1.9 MB of the checksum-finishing kernel.
MEASURED_TRAFFIC = {
    (2, 32, "k_gather"): 653.3e6, (2, 32, "k_scatter"): 4.8e6,
    (1, 2048, "k_gather"): 450.1e6, (1, 2048, "k_scatter"): 22.4e6,
    (3, 512, "k_gather"): 586.8e6, (3, 512, "k_scatter"): 934.9e6,
    (4, 8, "k_gather"): 661.3e6, (4, 8, "k_scatter"): 675.9e6,
    (5, 4, "k_gather"): 818.0e6, (5, 4, "k_scatter"): 548.6e6,
}
# the same for the reference's own 64-byte header (bench.py --ref64)
MEASURED_TRAFFIC_REF64 = {(2, 32, "k_gather"): 655.5e6, (2, 32, "k_scatter"): 4.8e6}
# The kernel sources those counter runs were made with (SHA-256).  A change to either file may change
# what the kernels move: `roofline.traffic` is then reported as null until the two counter passes have
# been run again and the figures above and these digests brought up to date (a CPU test holds them
# against the tree).
TRAFFIC_MEASURED_WITH = {
    "splitrpc_amd/csrc/sg_kernels_copy.h": "526d7000c8e7758c4accd6f38c4db3fcdb20738a7c8dbdd92c6877a1758de5f8",
    "splitrpc_amd/csrc/sg_device.h": "2e221986fd3ad868a696eb88ddc07a195d82b2e5b0fd4799e904894cc08aca4c",
}


def traffic_is_current() -> bool:
    """Whether the kernel sources are the ones MEASURED_TRAFFIC was measured with."""
    import hashlib
    here = os.path.dirname(os.path.abspath(__file__))
    for rel, digest in TRAFFIC_MEASURED_WITH.items():
        try:
            with open(os.path.join(here, rel), "rb") as f:
                if hashlib.sha256(f.read()).hexdigest() != digest:
                    return False
        except OSError:
            return False
    return True


WORKLOAD_NAMES = {1: "lenet", 2: "resnet50", 3: "bert", 4: "mixed", 5: "jumbo"}


def _log(msg: str) -> None:
    """Progress on stderr: a long run shows where it is."""
    print(f"[bench {time.perf_counter() - _T0:7.1f}s] {msg}", file=sys.stderr, flush=True)


_T0 = time.perf_counter()


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", type=int, default=2, help="1..5")
    ap.add_argument("--batches-per-launch", type=int, default=0,
                    help="batches laid side by side per call (0: default of the workload)")
    ap.add_argument("--rotate-mb", type=int, default=1024,
                    help="rotate over ring copies until the working set exceeds this many MB")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip requests/s of the other workloads")
    ap.add_argument("--ref64", action="store_true",
                    help="the reference's own 64-byte p2p_rpc_hdr (payload lengths from a table) instead of "
                         "the 58-byte benchmark header")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-remap", action="store_true", help="disable the XCD-aware launch order")
    ap.add_argument("--no-small", action="store_true",
                    help="one wavefront per frame even for short frames (SG_F_NO_SMALL)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 512 MiB device copy a few times (a kernel of known "
                         "traffic, to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    ap.add_argument("--one-stream", action="store_true",
                    help="gather and scatter calls on one context and stream (default: one each)")
    ap.add_argument("--no-single", action="store_true",
                    help="skip the single-batch legs (eager, HIP graphs on 1, 2 and 4 streams)")
    ap.add_argument("--general", action="store_true",
                    help="always run the descriptor pass (do not declare the fragmenting rule)")
    ap.add_argument("--leg", choices=["host-engine", "pipeline"], default=None,
                    help="run one leg alone and print its object (for a kernel trace of that leg): the C++ "
                         "engine's batched calls over P2pRpcRr objects, or the receive pipeline at whole-call bursts")
    ap.add_argument("--tx-in-order", action="store_true",
                    help="response frames take their TX slots in ring order (the generator's default "
                         "is a random permutation of the TX ring, the hardest order for the scatter)")
    return ap.parse_args()


DEFAULT_BPL = {1: 2048, 2: 32, 3: 512, 4: 8, 5: 4}


class Pool:
    """R device copies of one workload, rotated between steps."""

    def __init__(self, w, bpl: int, rotate_mb: int, extra_flags: int = 0, rule: bool = True):
        from splitrpc_amd.engine import DeviceWorkload
        per = (w.ring.nbytes + int(w.req_sizes.sum()) + w.tx_n_slots * w.slot_size
               + int(w.resp_sizes.sum())) * bpl
        r = max(2, min(64, -(-rotate_mb * (1 << 20) // max(per, 1))))
        self.items = [DeviceWorkload(w, copies=bpl, unique_tokens=True) for _ in range(r)]
        self.w = w
        self.bpl = bpl
        self.extra_flags = extra_flags
        self.rule = rule  # declare size + fragmenting rule where the workload has one size
        self.gather_bytes = w.gather_bytes() * bpl
        self.scatter_bytes = w.scatter_bytes() * bpl
        self.n_req = w.n_req * bpl

    def step(self, ctx, i: int, flags: int, ctx_tx=None) -> None:
        """One pass of the hot path.  With ctx_tx the scatter call goes to a
        second context on a stream of its own, as the reference keeps one copy
        context (and stream) per direction (src/p2p_rpc_sg_engine.h:185-196);
        an echo answered in place reads what its gather wrote and stays on one."""
        dw = self.items[i % len(self.items)]
        if ctx_tx is not None and self.w.tx_in_place:
            # An echo answered in place reads what its gather wrote and takes the descriptors that
            # gather built, so both calls of a step stay on one context; consecutive steps (other
            # rings, other arenas) take the two contexts in turns and overlap on their streams.
            c = ctx_tx if (i & 1) else ctx
            dw.gather(c, flags | self.extra_flags, rule=self.rule)
            dw.scatter(c, flags | self.extra_flags, fuse=self.rule, reuse=True)
            return
        dw.gather(ctx, flags | self.extra_flags, rule=self.rule)
        if ctx_tx is not None:
            dw.scatter(ctx_tx, flags | self.extra_flags, fuse=self.rule)
        else:
            # on one stream; an echo takes the descriptors its gather just built
            dw.scatter(ctx, flags | self.extra_flags, fuse=self.rule, reuse=True)


MIN_TIMED_MS = 50.0
# bursts of up to this many arrivals are reassembled in workgroups of 256 threads (SG_F_SMALL_GROUPS)
# where the reassembly runs beside a copy
BESIDE_UP_TO = 65536


def stat_line(ns) -> list:
    """[N, Mean, p90, p95, p99, min, max] of nanosecond samples, the summary the
    reference prints for its GDelay / SDelay vectors (print_stat,
    src/utils/stats_utils.h:69-79; a percentile is the sample at index
    round(p * (N - 1)) of the sorted samples, :10-21)."""
    v = sorted(int(x) for x in ns)
    if not v:
        return [0, 0.0, 0.0, 0.0, 0.0, 0, 0]
    pick = lambda p: float(v[int(round(p * (len(v) - 1)))])
    return [len(v), round(sum(v) / len(v), 2), pick(0.90), pick(0.95), pick(0.99), v[0], v[-1]]


class Timing(float):
    """Seconds per step (the median run, by the events on the streams), with
    what it was taken from."""
    host_clock = 0.0   # the same runs by the host's clock around a drain
    runs = 0
    timed_ms = 0.0


def timed(ctx, pool: Pool, steps: int, warmup: int, ctx_tx=None, reps: int = 5, min_ms: float = MIN_TIMED_MS,
          shunt: bool = False) -> Timing:
    """Seconds per step: `warmup` untimed steps, then timed runs of exactly
    `steps` steps each, every run bracketed by synchronization on both sides --
    at least `reps` runs and as many as it takes to have `min_ms` milliseconds
    timed in all (one run of 20 steps of 0.1 ms is a 2 ms sample).  A run is
    clocked twice: by events recorded on the streams the calls go to (the first
    before the run's first call, the last behind its last call on either
    stream), and by the host's clock around the run and the drain behind it.
    The median run by the events is the figure; the host clock's median, which
    carries the cost of the drain itself, rides along."""
    import torch
    from splitrpc_amd import capi

    streams = [torch.cuda.ExternalStream(c.stream, device="cuda:0") for c in (ctx, ctx_tx) if c is not None]

    def drain():
        ctx.sync()
        if ctx_tx is not None:
            ctx_tx.sync()
        torch.cuda.synchronize()

    def step(i):
        if shunt:
            pool.items[i % len(pool.items)].shunt(ctx, capi.F_ASYNC | pool.extra_flags, rule=pool.rule)
        else:
            pool.step(ctx, i, capi.F_ASYNC, ctx_tx)

    # every rotated copy is touched at least once before the clock starts
    for i in range(max(warmup, len(pool.items))):
        step(i)
    drain()
    ev_runs, host_runs, total = [], [], 0.0
    while len(ev_runs) < reps or total < min_ms * 1e-3:
        e0 = torch.cuda.Event(enable_timing=True)
        ends = [torch.cuda.Event(enable_timing=True) for _ in streams]
        t0 = time.perf_counter()
        e0.record(streams[0])
        for i in range(steps):
            step(warmup + i)
        for e, st in zip(ends, streams):
            e.record(st)
        drain()
        host = time.perf_counter() - t0
        ev = max(e0.elapsed_time(e) for e in ends) * 1e-3
        ev_runs.append(ev / steps)
        host_runs.append(host / steps)
        total += ev
        if len(ev_runs) >= 2000:
            break
    ev_runs.sort()
    host_runs.sort()
    t = Timing(ev_runs[len(ev_runs) // 2])
    t.host_clock = host_runs[len(host_runs) // 2]
    t.runs = len(ev_runs)
    t.timed_ms = total * 1e3
    return t


def kernel_times(ctx, pool: Pool, steps: int, shunt: bool = False):
    """Average duration of each kernel from HIP events recorded around every
    launch on the stream the kernels run on.  `shunt`: one launch per step that
    carries both directions (counted under k_gather)."""
    from splitrpc_amd import capi
    ctx.set_profiling(True)
    for i in range(steps):
        if shunt:
            pool.items[i % len(pool.items)].shunt(ctx, capi.F_ASYNC | pool.extra_flags, rule=pool.rule)
        else:
            pool.step(ctx, i, capi.F_ASYNC)
    out = {}
    for which, name in ((0, "k_prep"), (1, "k_gather"), (2, "k_scatter")):
        ms, n = ctx.kernel_time(which)
        out[name] = (ms / n if n else 0.0, n)
    ctx.set_profiling(False)
    return out


def _cpu_worker(w, seconds: float, n_copies: int, result: list, slot: int, start) -> None:
    """One shunter core: gather + scatter passes over its own rotated ring
    copies until the time is up.  The oracle's C calls release the GIL."""
    import dataclasses
    import numpy as np
    import oracle
    w = dataclasses.replace(w)  # private ring pointer
    rings = [w.ring.copy() for _ in range(n_copies)]
    txs = [w.tx_ring_init.copy() if w.tx_ring_init is not None else None for _ in range(n_copies)]
    src = w.resp_payload
    if w.out_tensor_sizes:
        rp = w.resp_payload.reshape(w.n_req, int(sum(w.out_tensor_sizes)))
        src, o = [], 0
        for s in w.out_tensor_sizes:
            src.append(np.ascontiguousarray(rp[:, o:o + s]).reshape(-1))
            o += s
    dst, _, _ = oracle.gather(w)  # destination reused by every pass
    start.wait()
    t0 = time.perf_counter()
    t_end = t0 + seconds
    it = 0
    while time.perf_counter() < t_end or it < 2:
        k = it % n_copies
        w.ring = rings[k]
        arena, _, _ = oracle.gather(w, out=dst)
        if w.tx_in_place:
            oracle.scatter(w, rings[k], rings[k], arena)
        else:
            oracle.scatter(w, rings[k], txs[k], src)
        it += 1
    result[slot] = (it, time.perf_counter() - t0)


def _cpu_run(w, seconds: float, threads: int):
    import threading
    n_copies = max(2, min(16, (512 << 20) // max(w.ring.nbytes * threads, 1)))
    result = [None] * threads
    start = threading.Barrier(threads)
    ts = [threading.Thread(target=_cpu_worker, args=(w, seconds, n_copies, result, i, start))
          for i in range(threads)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    passes = sum(r[0] for r in result)
    dt = max(r[1] for r in result)
    return passes, dt, n_copies


def back_to_back(ctx, pool: Pool, which: str, launches: int) -> float:
    """Seconds per launch of one kernel launched back to back: two HIP events on
    the context's stream around the whole burst (no event between launches, so
    the figure carries the gaps between kernels but not an event's own cost)."""
    import torch
    from splitrpc_amd import capi
    stream = torch.cuda.ExternalStream(ctx.stream, device="cuda:0")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n_items = len(pool.items)

    def launch(i):
        dw = pool.items[i % n_items]
        if which == "k_gather":
            dw.gather(ctx, capi.F_ASYNC | pool.extra_flags, rule=pool.rule)
        else:
            dw.scatter(ctx, capi.F_ASYNC | pool.extra_flags, fuse=pool.rule)

    for i in range(n_items):
        launch(i)
    ctx.sync()
    e0.record(stream)
    for i in range(launches):
        launch(i)
    e1.record(stream)
    e1.synchronize()
    ctx.sync()
    return e0.elapsed_time(e1) * 1e-3 / launches


def per_request_calls(ctx, dw, calls: int = 300):
    """The drop-in per-request path: one synchronous sg_hip_gather per request
    from a host-built run table, as copy_engine->gather(rr, stub) issues them
    (latency of table staging + launch + wait, one request at a time)."""
    import ctypes as C
    from splitrpc_amd import capi
    w = dw.w
    hl = 64 if w.profile == 1 else 58
    skbs = []
    for r in range(min(w.n_req, 8)):
        f0, f1 = int(w.req_first[r]), int(w.req_first[r + 1])
        skb = capi.SkBuf()
        off = 0
        for k, f in enumerate(range(f0, f1)):
            skb.i_buf[k] = dw.ring.data_ptr() + int(w.frag_slot[f]) * w.slot_size + hl
            skb.o_buf[k] = dw.req_arena.data_ptr() + r * int(w.req_sizes[r]) + off
            skb.len[k] = int(w.frag_len[f])
            off += int(w.frag_len[f])
        skb.num_items = f1 - f0
        skbs.append(skb)
    fn = ctx.lib.sg_hip_gather
    for i in range(20):
        assert fn(ctx.h, C.byref(skbs[i % len(skbs)])) == 0
    lat = []
    t0 = time.perf_counter()
    for i in range(calls):
        a = time.perf_counter_ns()
        fn(ctx.h, C.byref(skbs[i % len(skbs)]))
        lat.append(time.perf_counter_ns() - a)
    dt = (time.perf_counter() - t0) / calls
    size = int(w.req_sizes[0])
    return {"us_per_gather_call": round(dt * 1e6, 2), "runs_per_request": int(skbs[0].num_items),
            "request_bytes": size, "requests_per_sec": round(1.0 / dt, 1),
            "GBps": round((2 * size + 16 * int(skbs[0].num_items)) / dt / 1e9, 2),
            "latency_ns_[N,Mean,p90,p95,p99,min,max]": stat_line(lat)}


def native_loop_time(ctx, ctx_tx, pool: "Pool", steps: int):
    """Seconds per step when the loop that issues the calls is native code
    (sgh_step_loop_gpu of libsg_host.so: what a C++ shunter thread does, without
    the interpreter between the calls); the argument sets are the ones the
    Python loop has used."""
    import ctypes as C
    from splitrpc_amd import capi
    if pool.w.tx_in_place:
        return None
    host = C.CDLL(os.path.join(os.path.dirname(os.path.abspath(__file__)), "splitrpc_amd", "libsg_host.so"))
    fn = host.sgh_step_loop_gpu
    fn.restype = C.c_double
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32]
    tx = ctx_tx if ctx_tx is not None else ctx
    for i in range(len(pool.items)):
        pool.step(ctx, i, capi.F_ASYNC, ctx_tx)      # every item has its argument sets
    ctx.sync()
    tx.sync()
    gas = [next(v for k, v in dw._args.items() if k[0] == "g") for dw in pool.items]
    sas = [next(v for k, v in dw._args.items() if k[0] == "s") for dw in pool.items]
    n = len(pool.items)
    ga = (C.c_void_p * n)(*[C.addressof(a) for a in gas])
    sa = (C.c_void_p * n)(*[C.addressof(a) for a in sas])
    runs = []
    for rep in range(5):
        dt = fn(ctx.h, tx.h, ga, sa, n, steps)
        if dt < 0:
            raise RuntimeError(f"sgh_step_loop_gpu failed: {dt}")
        runs.append(dt / steps)
    runs.sort()
    return runs[len(runs) // 2]


def _host_lib():
    import ctypes as C
    host = C.CDLL(os.path.join(ROOT, "splitrpc_amd", "libsg_host.so"))
    host.sgh_shunt_loop_gpu.restype = C.c_double
    host.sgh_shunt_loop_gpu.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]
    host.sgh_engine_loop_gpu.restype = C.c_int
    host.sgh_engine_loop_gpu.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32,
                                         C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64,
                                         C.c_uint32, C.c_uint32, C.c_void_p, C.c_uint32, C.c_uint64, C.c_uint64,
                                         C.c_uint32, C.c_uint32, C.c_void_p]
    return host


def native_shunt_loop(ctxs, pool: "Pool", steps: int, latency: bool = False):
    """One sg_hip_shunt_batch call per step (both directions in one launch)
    from a native loop over `ctxs`, taken in turns so that len(ctxs) calls are
    in flight (sgh_shunt_loop_gpu of libsg_host.so).  Returns seconds per step
    (median of 5 loops); with `latency` (one context) every call is made
    synchronous and the calls' nanoseconds come back as well."""
    import ctypes as C
    import numpy as np
    from splitrpc_amd import capi
    if pool.w.tx_in_place:
        return None
    host = _host_lib()
    for dw in pool.items:
        dw.shunt(ctxs[0], capi.F_ASYNC | pool.extra_flags, rule=pool.rule)  # builds and keeps the argument sets
    ctxs[0].sync()
    gas = [next(v for k, v in dw._args.items() if k[0] == "g") for dw in pool.items]
    sas = [next(v for k, v in dw._args.items() if k[0] == "s") for dw in pool.items]
    for g_, s_ in zip(gas, sas):
        g_.flags |= capi.F_ASYNC
        s_.flags |= capi.F_ASYNC
    n = len(pool.items)
    ga = (C.c_void_p * n)(*[C.addressof(x) for x in gas])
    sa = (C.c_void_p * n)(*[C.addressof(x) for x in sas])
    hs = (C.c_void_p * len(ctxs))(*[c.h for c in ctxs])
    if latency:
        lat = np.zeros(steps, np.uint64)
        dt = host.sgh_shunt_loop_gpu(hs, 1, ga, sa, n, steps, lat.ctypes.data_as(C.c_void_p))
        if dt < 0:
            raise RuntimeError(f"sgh_shunt_loop_gpu failed: {dt}")
        return dt / steps, lat
    runs = []
    for rep in range(5):
        dt = host.sgh_shunt_loop_gpu(hs, len(ctxs), ga, sa, n, steps, None)
        if dt < 0:
            raise RuntimeError(f"sgh_shunt_loop_gpu failed: {dt}")
        runs.append(dt / steps)
    runs.sort()
    return runs[len(runs) // 2]


def host_engine_batched(pool: "Pool", steps: int, default_only: bool = False) -> dict:
    """The batched calls of the C++ drop-in, P2pRpcSgHipEngine::gather_batch(P2pRpcRr **) and
    scatter_batch(P2pRpcRr **), over the requests of one default call held as P2pRpcRr objects
    (sgh_engine_loop_gpu of libsg_host.so): with the engine walking every fragment on the host,
    and with the requests' fragment tables kept where the device reads them.  Response headers
    come from the connections' templates here (fresh response buffers, rr_set_hdr).  With the tables
    attached the engine decides per call: from 49152 fragments (frames) on the device pulls them,
    smaller calls' tables the calling thread walks and leaves in pinned memory for the kernels to
    read.  `default_only`: just that form (a call of another size than the default)."""
    import ctypes as C
    import numpy as np
    w = pool.w
    if w.in_tensor_sizes or w.out_tensor_sizes or w.tx_in_place or len(set(int(x) for x in w.req_sizes)) != 1:
        return None
    host = _host_lib()
    items = pool.items[:2]
    dw = items[0]
    bases = np.array([[d.ring.data_ptr(), d.tx_ring.data_ptr(), d.req_arena.data_ptr(), d.resp_arena.data_ptr()]
                      for d in items], np.uint64).reshape(-1)
    fs = np.ascontiguousarray(dw.frag_slot.cpu().numpy().view(np.uint32))
    fl = np.ascontiguousarray(dw.frag_len.cpu().numpy().view(np.uint32))
    ts = np.ascontiguousarray(dw.tx_slot.cpu().numpy().view(np.uint32))
    per, per_resp = dw.n_frags // dw.n_req, dw.n_frames // dw.n_req
    pv = lambda x: x.ctypes.data_as(C.c_void_p)
    out = {"requests": dw.n_req, "fragments": dw.n_frags, "response_frames": dw.n_frames}
    total = pool.gather_bytes + pool.scatter_bytes
    for mode, name in ((0, "tables_walked_by_the_host"), (1, "tables_pulled_by_the_device")):
        if default_only and mode == 0:
            continue
        res = np.zeros(16, np.float64)
        rc = host.sgh_engine_loop_gpu(0, mode, len(items), pv(bases), dw.rx.n_slots, w.slot_size, w.profile, pv(fs),
                                      pv(fl), dw.n_req, per, int(w.req_sizes[0]), dw.req_app.cap, w.mtu,
                                      dw.tx.n_slots, pv(ts), per_resp, int(w.resp_sizes[0]), dw.resp_app.cap,
                                      w.flags, steps, pv(res))
        if rc != 0:
            raise RuntimeError(f"sgh_engine_loop_gpu mode {mode} failed: {rc}")
        sec = float(res[0])
        out[name] = {"us_per_step": round(sec * 1e6, 2), "GBps": round(total / sec / 1e9, 1),
                     "frac_of_hbm_peak": round(total / sec / 1e9 / HBM_PEAK_GBS, 4),
                     "requests_per_sec": round(dw.n_req / sec, 1),
                     "host_us_per_gather_batch_call": round(float(res[2]) * 1e-3, 2),
                     "host_us_per_scatter_batch_call": round(float(res[9]) * 1e-3, 2),
                     "gather_batch_host_ns_[N,Mean,p90,p95,p99,min,max]": [round(float(x), 2) for x in res[1:8]],
                     "scatter_batch_host_ns_[N,Mean,p90,p95,p99,min,max]": [round(float(x), 2) for x in res[8:15]]}
    if default_only:
        return out["tables_pulled_by_the_device"]
    # the reference's own call through the same engine: one synchronous gather(rr, stub) per request
    res = np.zeros(16, np.float64)
    rc = host.sgh_engine_loop_gpu(0, 2, len(items), pv(bases), dw.rx.n_slots, w.slot_size, w.profile, pv(fs), pv(fl),
                                  dw.n_req, per, int(w.req_sizes[0]), dw.req_app.cap, w.mtu, dw.tx.n_slots, pv(ts),
                                  per_resp, int(w.resp_sizes[0]), dw.resp_app.cap, w.flags, 2000, pv(res))
    if rc != 0:
        raise RuntimeError(f"sgh_engine_loop_gpu mode 2 failed: {rc}")
    out["per_request_gather"] = {"us_per_call": round(float(res[0]) * 1e6, 2),
                                 "requests_per_sec": round(1.0 / float(res[0]), 1),
                                 "GDelay_ns_[N,Mean,p90,p95,p99,min,max]": [round(float(x), 2) for x in res[1:8]]}
    return out


def graph_step_time(w, extra: int, rule: bool, rotate_mb: int, steps: int = 16, replays: int = 50,
                    streams: int = 1, shunt: bool = False):
    """Seconds per step of the single-batch call when `steps` steps are recorded
    into one HIP graph per stream and the graphs are replayed: the launch-bound
    loop without the per-launch host cost.  With `streams` > 1 that many
    contexts, each with a stream, a graph and rings of its own, replay side by
    side (several batch-sized calls in flight at once); the figure is then wall
    time over ALL steps of all streams."""
    import torch
    from splitrpc_amd import capi
    from splitrpc_amd.engine import SgContext
    lanes = []
    for _ in range(streams):
        # every lane's stream on a hardware queue of its own where one is to be had: graphs replayed
        # on streams that share a queue run one after the other
        kw = dict(max_reqs=max(4096, w.n_req), max_frames=max(65536, w.n_frags, w.n_resp_frames))
        ctx = SgContext.apart_from([l[1] for l in lanes], 0, **kw) if lanes else SgContext(0, **kw)
        stream = torch.cuda.ExternalStream(ctx.stream, device="cuda:0")
        pool = Pool(w, 1, max(64, rotate_mb // streams), extra, rule=rule)

        def one(i, ctx=ctx, pool=pool):
            if shunt:
                pool.items[i % len(pool.items)].shunt(ctx, capi.F_ASYNC | pool.extra_flags, rule=pool.rule)
            else:
                pool.step(ctx, i, capi.F_ASYNC)

        for i in range(len(pool.items)):
            one(i)
        ctx.sync()
        lanes.append((stream, ctx, pool, one))
    torch.cuda.synchronize()
    graphs = []
    for stream, ctx, pool, one in lanes:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(steps):
                one(i)
        graphs.append(g)

    def replay_all():
        for (stream, _, _, _), g in zip(lanes, graphs):
            with torch.cuda.stream(stream):
                g.replay()

    for _ in range(3):
        replay_all()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(replays):
        replay_all()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / (replays * steps * streams)
    for _, ctx, _, _ in lanes:
        ctx.sync()
        ctx.close()
    return dt


def device_pipeline(pool: "Pool", calls: int = 6, bursts=(1024, 4096, 16384, 65536, 0), n_queues: int = 4,
                    queues_up_to: int = 1 << 30) -> dict:
    """The receive path end to end on the device, burst after burst and no
    host wait in between, from a native loop (sgh_pipeline_loop_gpu of
    libsg_host.so): sg_hip_reassemble files a burst's arrivals (requests that
    stay incomplete wait on the device), then the requests the burst completed
    are gathered and answered (their number stays on the device):
    sg_hip_shunt_batch, one launch for both directions where the burst is small
    enough, else a gather and a scatter call.  The stream of arrivals is that
    of `calls` default calls' worth of requests (the pool's ring copies in
    turns), in arrival order; wall time over the whole stream (burst 0 = a
    whole call's arrivals per burst).  Two forms:
      one_stream   the calls of a burst one after the other on one context
      overlapped   the reassembly on a context (stream) of its own, its output
                   tables double-buffered, events between the two streams: burst
                   k + 1 is filed while burst k is gathered and answered (in
                   workgroups of 256 threads, which find room beside the copy)
      N_queues     (bursts of up to `queues_up_to` arrivals) N receive queues side
                   by side, each a one_stream pipeline of its own (_pipeline_queues)"""
    import ctypes as C
    import numpy as np
    import torch
    from splitrpc_amd import capi
    from splitrpc_amd.engine import AppRef, RingRef, SgContext, to_dev
    w = pool.w
    if w.in_tensor_sizes or w.out_tensor_sizes or w.tx_in_place or len(set(int(x) for x in w.req_sizes)) != 1:
        return None
    host = _host_lib()
    host.sgh_pipeline_loop_gpu.restype = C.c_double
    host.sgh_pipeline_loop_gpu.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_int]
    host.sgh_pipeline_queues_gpu.restype = C.c_double
    host.sgh_pipeline_queues_gpu.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                             C.c_int]
    dev = "cuda:0"
    items = pool.items
    dw = items[0]
    # ring copies for the queues of the side-by-side form: no two queues on one copy at a time
    from splitrpc_amd.engine import DeviceWorkload
    items_q = list(items) + [DeviceWorkload(w, copies=pool.bpl, unique_tokens=True)
                             for _ in range(max(0, n_queues - len(items)))]
    size, rsize = int(w.req_sizes[0]), int(w.resp_sizes[0])
    per, per_resp = -(-size // w.mtu), -(-rsize // w.mtu)
    n_arr = int(dw.arrivals.numel())
    out = {"arrivals_per_call": n_arr, "requests_per_call": dw.n_req, "calls": calls}
    # position in the arrival stream of every request's last fragment (the batch's order, tiled over the call)
    at = np.empty(w.n_slots, np.int64)
    at[w.arrivals] = np.arange(w.n_frags)
    last = np.array([at[w.frag_slot[int(w.req_first[r]):int(w.req_first[r + 1])]].max() for r in range(w.n_req)])
    done_at = np.concatenate([last + i * w.n_frags for i in range(n_arr // w.n_frags)])
    total_bytes = (pool.gather_bytes + pool.scatter_bytes) * calls
    for burst in bursts:
        burst = burst or n_arr
        if burst > n_arr:
            continue
        # requests a burst can complete: a request is complete with its last arrival, and arrival
        # orders that interleave the requests of a batch complete many of them within one burst
        bound = int(np.bincount(done_at // burst).max())
        mf = max(65536, bound * per, burst)
        ctx_sg = SgContext(0, max_reqs=max(4096, dw.n_req), max_frames=mf)
        ctx_ra = SgContext.apart_from([ctx_sg], 0, max_reqs=max(4096, dw.n_req), max_frames=mf)  # another hardware queue
        i32 = lambda n: torch.zeros(n, dtype=torch.int32, device=dev)
        # reassembly output, twice: while the copy reads one set the next burst fills the other
        sets = [dict(fs=i32(mf), fl=i32(mf), rf=i32(4097 + dw.n_req), hdr=i32(4096 + dw.n_req), counts=i32(4))
                for _ in range(2)]
        req_cap, resp_cap = 4 * bound * size, 4 * bound * rsize
        req_arena = torch.zeros(req_cap, dtype=torch.uint8, device=dev)
        resp_arena = torch.zeros(resp_cap, dtype=torch.uint8, device=dev)
        tx_ring = torch.zeros(bound * per_resp * w.slot_size, dtype=torch.uint8, device=dev)
        tx = RingRef(tx_ring, bound * per_resp, w.slot_size, w.profile)
        tx_slot = to_dev(np.arange(bound * per_resp, dtype=np.uint32), dev)
        resp_first = to_dev((np.arange(bound + 1) * per_resp).astype(np.uint32), dev)
        A = capi.F_ASYNC
        # ras_beside: the same calls in workgroups of 256 threads, for the form whose reassembly runs beside the copy
        ras, ras_beside, gas, sas = [], [], [], []
        by_item = {}
        for call in range(calls):
            it = items[call % len(items)]
            for b in range(0, n_arr, burst):
                j = len(ras) & 1
                t = sets[j]
                key = (call % len(items), j)
                if key not in by_item:
                    by_item[key] = (
                        ctx_sg.gather_args(it.rx, t["fs"], None, t["rf"], bound, bound * per,
                                           AppRef(arena=req_arena, cap=req_cap), None, flags=A | capi.F_RULE_FRAGS,
                                           fixed_req_size=size, mtu=w.mtu, counts=t["counts"]),
                        ctx_sg.scatter_args(it.rx, tx, tx_slot, None, resp_first, None, rsize, bound, bound * per_resp,
                                            w.mtu, AppRef(arena=resp_arena, cap=resp_cap), None, w.flags | A,
                                            hdr_src_req=t["hdr"], counts=t["counts"]))
                for lst, fl_ in ((ras, A), (ras_beside, A | capi.F_SMALL_GROUPS)):
                    lst.append(ctx_sg.reassemble_args(it.rx, it.arrivals[b:b + burst], min(burst, n_arr - b), t["fs"],
                                                      t["fl"], t["rf"], req_hdr_slot=t["hdr"], counts_out=t["counts"],
                                                      flags=fl_))
                gas.append(by_item[key][0])
                sas.append(by_item[key][1])
        n_bursts = len(ras)
        arr = lambda xs: (C.c_void_p * len(xs))(*[C.addressof(x) for x in xs])
        c_ras, c_ras_beside, c_gas, c_sas = arr(ras), arr(ras_beside), arr(gas), arr(sas)
        res = {}
        for form in ("one_stream", "overlapped"):
            c_ra = ctx_sg if form == "one_stream" else ctx_ra
            best = None
            for rep in range(3):
                c_ra.reassemble_reset()
                torch.cuda.synchronize()
                beside = form == "overlapped" and burst <= BESIDE_UP_TO
                dt = host.sgh_pipeline_loop_gpu(c_ra.h, ctx_sg.h, c_ras_beside if beside else c_ras,
                                                c_gas, c_sas, n_bursts, 1 if form == "overlapped" else 0)
                if dt < 0:
                    raise RuntimeError(f"sgh_pipeline_loop_gpu failed: {dt} {ctx_sg.lib.sg_hip_last_error(ctx_sg.h)}")
                best = dt if best is None else min(best, dt)
            left = int(sets[(n_bursts - 1) & 1]["counts"].cpu()[3])
            res[form] = {"us_per_burst": round(best / n_bursts * 1e6, 2),
                         "arrivals_per_sec": round(n_arr * calls / best, 1),
                         "requests_per_sec": round(dw.n_req * calls / best, 1),
                         "payload_Gbit_per_sec": round(8.0 * size * dw.n_req * calls / best / 1e9, 1),
                         "GBps": round(total_bytes / best / 1e9, 1),
                         "frac_of_hbm_peak": round(total_bytes / best / 1e9 / HBM_PEAK_GBS, 4),
                         "requests_left_in_flight": left}
        out[str(burst)] = res
        ctx_ra.close()
        ctx_sg.close()
        del sets, req_arena, resp_arena, tx_ring, gas, sas, ras, ras_beside, by_item
        torch.cuda.empty_cache()
        if burst <= queues_up_to:
            res[f"{n_queues}_queues"] = _pipeline_queues(host, pool, items_q, n_queues, calls, burst, bound, mf, size,
                                                         rsize, per, per_resp, n_arr, total_bytes)
    return out


def _pipeline_queues(host, pool, items, n_queues, calls, burst, bound, mf, size, rsize, per, per_resp, n_arr,
                     total_bytes) -> dict:
    """`n_queues` receive queues side by side, each the one-stream pipeline of
    device_pipeline with a context (stream on a hardware queue of its own where
    one is to be had, reassembly table, cursors), tables, arenas and TX ring of
    its own, each fed `calls` calls' worth of arrivals from ring copies no other
    queue is on at the time (sgh_pipeline_queues_gpu: one thread queues burst k
    of every queue, then burst k + 1; or a thread per queue).  Wall time over
    all queues' arrivals."""
    import ctypes as C
    import numpy as np
    import torch
    from splitrpc_amd import capi
    from splitrpc_amd.engine import AppRef, RingRef, SgContext, to_dev
    w = pool.w
    dev = "cuda:0"
    dw = items[0]
    A = capi.F_ASYNC
    i32 = lambda n: torch.zeros(n, dtype=torch.int32, device=dev)
    # a queue's reassembly runs beside the other queues' copies: workgroups of 256 threads -- up to
    # bursts of 65536 arrivals; a whole call's reassembly takes slots from the copy for longer than it
    # gains by not waiting for the copy's end (130 us per burst with workgroups of 1024 threads, 137 with 256)
    ra_flags = capi.F_SMALL_GROUPS if burst <= BESIDE_UP_TO else 0
    ctxs, keep, ras, gas, sas = [], [], [], [], []
    for q in range(n_queues):
        kw = dict(max_reqs=max(4096, dw.n_req), max_frames=mf)
        ctx = SgContext.apart_from(ctxs, 0, **kw) if ctxs else SgContext(0, **kw)
        ctxs.append(ctx)
        t = dict(fs=i32(mf), fl=i32(mf), rf=i32(4097 + dw.n_req), hdr=i32(4096 + dw.n_req), counts=i32(4))
        req_cap, resp_cap = 4 * bound * size, 4 * bound * rsize
        req_arena = torch.zeros(req_cap, dtype=torch.uint8, device=dev)
        resp_arena = torch.zeros(resp_cap, dtype=torch.uint8, device=dev)
        tx_ring = torch.zeros(bound * per_resp * w.slot_size, dtype=torch.uint8, device=dev)
        tx = RingRef(tx_ring, bound * per_resp, w.slot_size, w.profile)
        tx_slot = to_dev(np.arange(bound * per_resp, dtype=np.uint32), dev)
        resp_first = to_dev((np.arange(bound + 1) * per_resp).astype(np.uint32), dev)
        keep.append((t, req_arena, resp_arena, tx_ring, tx_slot, resp_first))
        by_item = {}
        for call in range(calls):
            k = (call + q) % len(items)
            it = items[k]
            if k not in by_item:
                by_item[k] = (
                    ctx.gather_args(it.rx, t["fs"], None, t["rf"], bound, bound * per,
                                    AppRef(arena=req_arena, cap=req_cap), None, flags=A | capi.F_RULE_FRAGS,
                                    fixed_req_size=size, mtu=w.mtu, counts=t["counts"]),
                    ctx.scatter_args(it.rx, tx, tx_slot, None, resp_first, None, rsize, bound, bound * per_resp,
                                     w.mtu, AppRef(arena=resp_arena, cap=resp_cap), None, w.flags | A,
                                     hdr_src_req=t["hdr"], counts=t["counts"]))
            for b in range(0, n_arr, burst):
                ras.append(ctx.reassemble_args(it.rx, it.arrivals[b:b + burst], min(burst, n_arr - b), t["fs"], t["fl"],
                                               t["rf"], req_hdr_slot=t["hdr"], counts_out=t["counts"],
                                               flags=A | ra_flags))
                gas.append(by_item[k][0])
                sas.append(by_item[k][1])
    n_bursts = len(ras) // n_queues
    arr = lambda xs: (C.c_void_p * len(xs))(*[C.addressof(x) for x in xs])
    c_ctx = (C.c_void_p * n_queues)(*[c.h for c in ctxs])
    c_ras, c_gas, c_sas = arr(ras), arr(gas), arr(sas)
    hw = len(set(c.stream_queue() for c in ctxs))
    res = {"hardware_queues": hw}
    for form, threaded in (("one_thread", 0), ("thread_per_queue", 1)):
        best = None
        for rep in range(3):
            for c in ctxs:
                c.reassemble_reset()
            torch.cuda.synchronize()
            dt = host.sgh_pipeline_queues_gpu(c_ctx, n_queues, c_ras, c_gas, c_sas, n_bursts, threaded)
            if dt < 0:
                raise RuntimeError(f"sgh_pipeline_queues_gpu failed: {dt} {[c.lib.sg_hip_last_error(c.h) for c in ctxs]}")
            best = dt if best is None else min(best, dt)
        left = sum(int(k[0]["counts"].cpu()[3]) for k in keep)
        res[form] = {"us_per_burst": round(best / (n_bursts * n_queues) * 1e6, 2),
                     "arrivals_per_sec": round(n_arr * calls * n_queues / best, 1),
                     "requests_per_sec": round(dw.n_req * calls * n_queues / best, 1),
                     "payload_Gbit_per_sec": round(8.0 * size * dw.n_req * calls * n_queues / best / 1e9, 1),
                     "GBps": round(total_bytes * n_queues / best / 1e9, 1),
                     "frac_of_hbm_peak": round(total_bytes * n_queues / best / 1e9 / HBM_PEAK_GBS, 4),
                     "requests_left_in_flight": left}
    for c in ctxs:
        c.close()
    del keep, ras, gas, sas
    torch.cuda.empty_cache()
    return res


def roofline_of(pool: Pool, kt, traffic_known: bool = True) -> dict:
    """Both copy kernels of a workload against the HBM peak: algorithmic bytes
    per call over the average duration of the call's copy kernels (HIP events
    around each launch on the stream they run on)."""
    out = {}
    for name, nbytes in (("k_gather", pool.gather_bytes), ("k_scatter", pool.scatter_bytes)):
        ms = kt[name][0]
        gbps = nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
        out[name] = {"avg_kernel_us": round(ms * 1e3, 3), "bytes_per_launch": nbytes, "GBps": round(gbps, 1),
                     "frac": round(gbps / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get((pool.w.cfg, pool.bpl, name)) if traffic_known else None}
    return out


def cpu_baseline(w, seconds: float):
    """The CPU oracle (a restatement of the reference's CPU scatter-gather
    path) timed on this host over rotated ring copies: on one thread -- the
    reference runs gather and scatter on one shunter core -- and on one thread
    per core of this job's CPU share, each thread taking whole batches."""
    bytes_per = w.gather_bytes() + w.scatter_bytes()
    it, dt, n_copies = _cpu_run(w, seconds * 0.6, 1)
    out = {"value": round(bytes_per * it / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
           "requests_per_sec": round(w.n_req * it / dt, 1),
           "sample": f"{it} passes of gather+scatter over one {w.name} batch "
                     f"({w.n_req} requests), {n_copies} rotated ring copies, {dt:.1f} s, "
                     "C oracle -O3, one thread"}
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    cores = max(1, min(cores, 16))
    if cores > 1:
        it, dt, n_copies = _cpu_run(w, seconds * 0.4, cores)
        out["all_cores"] = {"value": round(bytes_per * it / dt / 1e9, 3), "unit": "GB/s", "cores": cores,
                            "requests_per_sec": round(w.n_req * it / dt, 1),
                            "sample": f"{it} passes in {dt:.1f} s, one thread per core, each thread its own "
                                      f"batches and {n_copies} rotated ring copies"}
    return out


def main() -> int:
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        return 2
    import torch
    from splitrpc_amd import capi, synth
    from splitrpc_amd.engine import SgContext

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (cuda:0)", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    # no collector pauses inside timed loops (a full collection over this process's objects takes
    # tens of milliseconds, and a loop of a few hundred microsecond-sized calls can trigger one)
    import gc
    gc.disable()
    extra = (capi.F_NO_XCD_REMAP if a.no_remap else 0) | (capi.F_NO_SMALL if a.no_small else 0)
    bpl = a.batches_per_launch or DEFAULT_BPL[a.workload]
    prof = synth.HDR_REF64 if a.ref64 else synth.HDR_BL58
    w = synth.make_workload(a.workload, profile=prof)
    if a.tx_in_order and not w.tx_in_place:
        import numpy as np
        w.tx_slot = np.sort(w.tx_slot)
    rule = not a.general

    def contexts(wl, b):
        mr, mf = max(4096, wl.n_req * b), max(65536, max(wl.n_frags, wl.n_resp_frames) * b)
        # gather and scatter each on a context (and stream) of their own, unless one stream is asked for; the
        # second stream on another hardware queue than the first, or the two would never run side by side
        c0 = SgContext(0, max_reqs=mr, max_frames=mf)
        return c0, (None if a.one_stream else SgContext.apart_from([c0], 0, max_reqs=mr, max_frames=mf))

    ctx, ctx_tx = contexts(w, bpl)
    _log(f"staging {w.name} x {bpl} batches per launch")
    pool = Pool(w, bpl, a.rotate_mb, extra, rule=rule)
    _log(f"{len(pool.items)} ring copies staged")

    if a.leg:
        res = host_engine_batched(pool, max(20, min(a.steps, 200))) if a.leg == "host-engine" else \
            device_pipeline(pool, calls=4, bursts=(65536, 0))
        print(json.dumps({a.leg: res}))
        ctx.close()
        if ctx_tx is not None:
            ctx_tx.close()
        return 0

    if a.calib_copy:
        src = torch.empty(512 << 20, dtype=torch.uint8, device="cuda:0").fill_(3)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    sec = timed(ctx, pool, a.steps, a.warmup, ctx_tx)
    _log(f"timed: {sec * 1e6:.1f} us per step by the streams' events, {sec.host_clock * 1e6:.1f} us by the host clock "
         f"(medians of {sec.runs} runs of {a.steps} steps, {sec.timed_ms:.1f} ms timed)")
    kt = kernel_times(ctx, pool, min(a.steps, 100))
    total_bytes = pool.gather_bytes + pool.scatter_bytes
    value = total_bytes / sec / 1e9
    dom = "k_gather" if pool.gather_bytes >= pool.scatter_bytes else "k_scatter"
    dom_bytes = pool.gather_bytes if dom == "k_gather" else pool.scatter_bytes
    dom_ms = kt[dom][0]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9 if dom_ms > 0 else 0.0
    b2b = back_to_back(ctx, pool, dom, min(a.steps, 100))
    # the counters were read with the default kernels and headers only
    traffic_known = not (a.general or a.ref64 or a.no_small or a.no_remap) and traffic_is_current()
    headline_roofs = roofline_of(pool, kt, traffic_known)

    _log("kernel times and back-to-back done; reassembly")
    # request reassembly on the device for the same call's arrivals (synchronous: counts come back)
    dw0 = pool.items[0]
    n_arr = int(dw0.arrivals.numel())
    ra_fs = torch.zeros(n_arr, dtype=torch.int32, device="cuda:0")
    ra_fl = torch.zeros(n_arr, dtype=torch.int32, device="cuda:0")
    ra_rf = torch.zeros(pool.n_req + 1, dtype=torch.int32, device="cuda:0")
    ra_kw = {}
    if a.ref64:
        # the reference's header carries no lengths: they come per slot, as from the NIC, and a
        # request is complete when its bytes add up to the server-wide request size
        ln = torch.zeros(int(dw0.rx.n_slots), dtype=torch.int32, device="cuda:0")
        ln[dw0.frag_slot.long()] = dw0.frag_len
        ra_kw = {"len_nic": ln, "req_size": int(w.req_sizes[0])}
    for _ in range(3):
        got = ctx.reassemble(dw0.rx, dw0.arrivals, n_arr, ra_fs, ra_fl, ra_rf, **ra_kw)
    t0 = time.perf_counter()
    for _ in range(20):
        got = ctx.reassemble(dw0.rx, dw0.arrivals, n_arr, ra_fs, ra_fl, ra_rf, **ra_kw)
    ra_sec = (time.perf_counter() - t0) / 20
    reassembly = {"arrivals": n_arr, "requests": got[0], "ms_per_call": round(ra_sec * 1e3, 4),
                  "arrivals_per_sec": round(n_arr / ra_sec, 1),
                  "tables_match_pre_staged": bool(got[0] == pool.n_req and torch.equal(ra_fs, dw0.frag_slot))}
    # the same arrivals in bursts of 64, as a NIC delivers them: incomplete requests stay on the device
    n_b = min(n_arr, 64 * 200)
    for b in range(0, n_b, 64):
        ctx.reassemble(dw0.rx, dw0.arrivals[b:b + 64], min(64, n_b - b), ra_fs, ra_fl, ra_rf, **ra_kw)
    ctx.reassemble_reset()
    lat = []
    t0 = time.perf_counter()
    for b in range(0, n_b, 64):
        t1 = time.perf_counter_ns()
        ctx.reassemble(dw0.rx, dw0.arrivals[b:b + 64], min(64, n_b - b), ra_fs, ra_fl, ra_rf, **ra_kw)
        lat.append(time.perf_counter_ns() - t1)
    reassembly["us_per_burst_of_64"] = round((time.perf_counter() - t0) / max(1, (n_b + 63) // 64) * 1e6, 2)
    reassembly["burst_of_64_latency_ns_[N,Mean,p90,p95,p99,min,max]"] = stat_line(lat)
    ctx.reassemble_reset()
    # the same bursts queued without waiting for each one's counts (they stay on the device, where the
    # gather reads them): what a burst costs the stream
    queued = [ctx.reassemble_args(dw0.rx, dw0.arrivals[b:b + 64], min(64, n_b - b), ra_fs, ra_fl, ra_rf,
                                  flags=capi.F_ASYNC, **ra_kw) for b in range(0, n_b, 64)]
    for qa in queued[:8]:
        ctx.reassemble_raw(qa)
    ctx.sync()
    ctx.reassemble_reset()
    t0 = time.perf_counter()
    for k, qa in enumerate(queued):
        ctx.reassemble_raw(qa)
        if k % 100 == 99:
            ctx.sync()  # a caller takes the counts in now and then
    ctx.sync()
    reassembly["us_per_burst_of_64_queued"] = round((time.perf_counter() - t0) / max(1, len(queued)) * 1e6, 2)
    ctx.reassemble_reset()
    del ra_fs, ra_fl, ra_rf
    _log("device pipeline")
    pipeline = device_pipeline(pool) if not a.ref64 else None

    # how the dominant kernel and the whole step scale with the batches laid side by side in one call
    by_bpl = {}
    if not a.no_sweep:
        _log("batches-per-launch sweep")
        for b in (1, 2, 4, 8, 16, 32):
            if b == bpl:
                by_bpl[str(b)] = {"ms_per_step": round(sec * 1e3, 5), "GBps": round(value, 1),
                                  "kernel": dom, "avg_kernel_us": round(dom_ms * 1e3, 3),
                                  "frac": round(achieved / HBM_PEAK_GBS, 4)}
                continue
            pb = Pool(w, b, a.rotate_mb, extra, rule=rule)
            sb = timed(ctx, pb, max(20, a.steps // 4), max(5, a.warmup // 4), ctx_tx, reps=3)
            kb = kernel_times(ctx, pb, 50)
            nb = pb.gather_bytes if dom == "k_gather" else pb.scatter_bytes
            gb = nb / (kb[dom][0] * 1e-3) / 1e9 if kb[dom][0] > 0 else 0.0
            by_bpl[str(b)] = {"ms_per_step": round(sb * 1e3, 5),
                              "GBps": round((pb.gather_bytes + pb.scatter_bytes) / sb / 1e9, 1),
                              "kernel": dom, "avg_kernel_us": round(kb[dom][0] * 1e3, 3),
                              "frac": round(gb / HBM_PEAK_GBS, 4)}
            del pb
            torch.cuda.empty_cache()

    _log("single-batch call")
    # the single-batch call of the same workload -- the call BASELINE's config words literally
    single = None
    if bpl != 1 and not a.no_single:
        p1 = Pool(w, 1, a.rotate_mb, extra, rule=rule)
        b1 = p1.gather_bytes + p1.scatter_bytes

        def fig(sec_per_step):
            return {"us_per_step": round(sec_per_step * 1e6, 3), "GBps": round(b1 / sec_per_step / 1e9, 1),
                    "frac_of_hbm_peak": round(b1 / sec_per_step / 1e9 / HBM_PEAK_GBS, 4),
                    "requests_per_sec": round(p1.n_req / sec_per_step, 1)}

        # two calls per step, a context (stream) per direction
        s1 = timed(ctx, p1, a.steps, a.warmup, ctx_tx)
        k1 = kernel_times(ctx, p1, min(a.steps, 100))
        single = {"ms_per_step": round(s1 * 1e3, 5), "GBps": round(b1 / s1 / 1e9, 2),
                  "requests_per_sec": round(p1.n_req / s1, 1),
                  "kernel_us": {k: round(v[0] * 1e3, 3) for k, v in k1.items()},
                  "k_gather_GBps": round(p1.gather_bytes / (k1["k_gather"][0] * 1e-3) / 1e9, 1)
                  if k1["k_gather"][0] > 0 else None}
        nl = native_loop_time(ctx, ctx_tx, p1, max(a.steps, 200))
        if nl is not None:
            single["native_loop_ms_per_step"] = round(nl * 1e3, 5)
            single["native_loop_GBps"] = round(b1 / nl / 1e9, 1)
            single["native_loop_requests_per_sec"] = round(p1.n_req / nl, 1)
        if not w.tx_in_place:
            # one call and ONE launch per step (sg_hip_shunt_batch: the scatter's frames ride in the gather's grid)
            ks = kernel_times(ctx, p1, min(a.steps, 100), shunt=True)
            one = {"python_loop_one_stream": fig(timed(ctx, p1, a.steps, a.warmup, None, shunt=True)),
                   "kernel_us": round(ks["k_gather"][0] * 1e3, 3),
                   "kernel_frac_of_hbm_peak": round(b1 / (ks["k_gather"][0] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
                   if ks["k_gather"][0] > 0 else None}
            more = []
            for _ in range(3):
                more.append(SgContext.apart_from([ctx] + more, 0, max_reqs=4096, max_frames=65536))
            n_native = max(a.steps, 400)
            for n_ctx in (1, 2, 4):
                one[f"native_loop_{n_ctx}_stream{'s' if n_ctx > 1 else ''}"] = fig(
                    native_shunt_loop(([ctx] + more)[:n_ctx], p1, n_native))
            dt, lat = native_shunt_loop([ctx], p1, 1000, latency=True)
            one["synchronous_call"] = {"us_per_call": round(dt * 1e6, 2),
                                       "latency_ns_[N,Mean,p90,p95,p99,min,max]": stat_line(lat)}
            for c in more:
                c.close()
            single["one_launch_per_step"] = one
        del p1
        for n_streams in (1, 2, 4):
            sg = graph_step_time(w, extra, rule, a.rotate_mb, streams=n_streams)
            key = "hip_graph" if n_streams == 1 else f"hip_graph_{n_streams}_streams"
            single[key + "_ms_per_step"] = round(sg * 1e3, 5)
            single[key + "_GBps"] = round(b1 / sg / 1e9, 1)
            single[key + "_requests_per_sec"] = round(w.n_req / sg, 1)
            if not w.tx_in_place:
                sg = graph_step_time(w, extra, rule, a.rotate_mb, streams=n_streams, shunt=True)
                single["one_launch_per_step"][key] = {
                    "us_per_step": round(sg * 1e6, 3), "GBps": round(b1 / sg / 1e9, 1),
                    "frac_of_hbm_peak": round(b1 / sg / 1e9 / HBM_PEAK_GBS, 4),
                    "requests_per_sec": round(w.n_req / sg, 1)}
            torch.cuda.empty_cache()

    host_engine = None
    if not a.no_single:
        _log("C++ engine, batched calls over P2pRpcRr objects")
        host_engine = host_engine_batched(pool, max(50, min(a.steps, 200)))
        if host_engine is not None and bpl != 1:
            # one batch per call, as the reference's shunter makes them: tables attached, the engine's choice
            p1 = Pool(w, 1, 128, extra, rule=rule)
            host_engine["single_batch_call"] = host_engine_batched(p1, 500, default_only=True)
            del p1
            torch.cuda.empty_cache()

    _log("per-request calls")
    per_req = per_request_calls(ctx, pool.items[0]) if not w.in_tensor_sizes else None
    rps = {WORKLOAD_NAMES[a.workload]: round(pool.n_req / sec, 1)}
    sweep = {}
    if not a.no_sweep:
        for cfg in (1, 2, 3, 4, 5):
            if cfg == a.workload:
                continue
            wc = synth.make_workload(cfg)
            b = DEFAULT_BPL[cfg]
            _log(f"sweep: {wc.name} x {b}")
            c2, c2_tx = contexts(wc, b)
            pc = Pool(wc, b, a.rotate_mb, extra, rule=rule)
            sc = timed(c2, pc, a.steps, a.warmup, c2_tx)
            kc = kernel_times(c2, pc, 50)
            tb = pc.gather_bytes + pc.scatter_bytes
            forms = {"two_calls": {"ms_per_step": round(sc * 1e3, 5), "GBps": round(tb / sc / 1e9, 2),
                                   "frac_of_hbm_peak": round(tb / sc / 1e9 / HBM_PEAK_GBS, 4)}}
            step_call = "two_calls"
            if not (wc.tx_in_place or wc.in_tensor_sizes or wc.out_tensor_sizes):
                # the same step as ONE call (sg_hip_shunt_batch): one launch where the two halves can share one
                so = timed(c2, pc, a.steps, a.warmup, None, shunt=True)
                ko = kernel_times(c2, pc, 50, shunt=True)
                forms["one_call"] = {"ms_per_step": round(so * 1e3, 5), "GBps": round(tb / so / 1e9, 2),
                                     "frac_of_hbm_peak": round(tb / so / 1e9 / HBM_PEAK_GBS, 4),
                                     "launches_per_step": int(sum(v[1] for v in ko.values()) // 50),
                                     "kernel_us": {k: round(v[0] * 1e3, 3) for k, v in ko.items() if v[1]}}
                if so < sc:
                    sc, step_call = so, "one_call"
            rps[wc.name] = round(pc.n_req / sc, 1)
            sweep[wc.name] = {"batches_per_launch": b, "ms_per_step": round(sc * 1e3, 5),
                              "GBps": round(tb / sc / 1e9, 2),
                              "frac_of_hbm_peak": round(tb / sc / 1e9 / HBM_PEAK_GBS, 4),
                              # the faster of the two ways to issue a step: a gather call and a scatter call on a
                              # stream each, or both as one sg_hip_shunt_batch call
                              "step_call": step_call, "step_forms": forms,
                              "kernels": roofline_of(pc, kc, traffic_known)}
            del pc
            if cfg == 5 and not a.tx_in_order:
                # the same responses into TX slots taken in ring order (the default is a random
                # permutation of the TX ring, which costs the scatter a tenth)
                import numpy as np
                wc.tx_slot = np.sort(wc.tx_slot)
                po = Pool(wc, b, a.rotate_mb, extra, rule=rule)
                timed(c2, po, 20, 5, c2_tx, reps=1)
                ko = kernel_times(c2, po, 50)
                sweep[wc.name]["tx_slots_in_ring_order"] = roofline_of(po, ko, False)["k_scatter"]
                del po
            c2.close()
            if c2_tx is not None:
                c2_tx.close()
            torch.cuda.empty_cache()

    if not a.no_sweep and not a.ref64:
        # the headline workload again with the reference's own 64-byte header
        wr = synth.make_workload(a.workload, profile=synth.HDR_REF64)
        pr = Pool(wr, bpl, a.rotate_mb, extra, rule=rule)
        sr = timed(ctx, pr, a.steps, a.warmup, ctx_tx)
        kr = kernel_times(ctx, pr, 50)
        roofs = roofline_of(pr, kr, False)
        for name in roofs:
            roofs[name]["traffic"] = MEASURED_TRAFFIC_REF64.get((a.workload, bpl, name)) if traffic_known else None
        sweep[wr.name + "_ref64_headers"] = {"batches_per_launch": bpl, "ms_per_step": round(sr * 1e3, 5),
                                             "GBps": round((pr.gather_bytes + pr.scatter_bytes) / sr / 1e9, 2),
                                             "frac_of_hbm_peak": round((pr.gather_bytes + pr.scatter_bytes) / sr / 1e9
                                                                       / HBM_PEAK_GBS, 4),
                                             "kernels": roofs}
        del pr

    out = {
        "metric": "gather+scatter GB/s (algorithmic bytes) on 1 MI355X",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(sec * 1e3, 5),
        "ms_per_step_host_clock": round(sec.host_clock * 1e3, 5),
        "timed_runs": sec.runs,
        "timed_ms": round(sec.timed_ms, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: {w.n_req} requests x {int(w.req_sizes[0])} B in "
                               f"{w.n_frags // w.n_req} frames of <= {w.mtu} B, {w.slot_size}-B slots, "
                               f"{w.n_resp_frames // w.n_req} response frames per request",
                   "batches_per_launch": bpl, "rotated_ring_copies": len(pool.items),
                   "requests_per_step": pool.n_req, "header_profile": "REF64" if a.ref64 else "BL58",
                   "descriptor_pass": "general (prefix scan)" if a.general else
                   "fused where the workload has one size (fragmenting rule declared and checked)",
                   "streams": "one" if a.one_stream else
                   "both calls of a step on one context (the echo reads what its gather wrote), consecutive "
                   "steps on two contexts and streams in turns" if w.tx_in_place else
                   "gather and scatter calls on a stream each (a copy context per direction)",
                   "timing": f"median of {sec.runs} runs of {a.steps} steps each ({sec.timed_ms:.0f} ms timed), every run "
                             "between synchronization on both sides; a run is clocked by events on the streams "
                             "(ms_per_step, value) and by the host clock around the run and its drain "
                             "(ms_per_step_host_clock)", "flags": w.flags,
                   "tx_slots": "ring order" if a.tx_in_order else "random permutation of the TX ring"},
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "requests_per_sec": rps,
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get((a.workload, bpl, dom)) if traffic_known else None,
                     "traffic_unit": "HBM bytes per launch (rocprofv3 --pmc, see profiles/)"
                                     if traffic_is_current() else
                                     "null: the kernel sources have changed since the counter runs (TRAFFIC_MEASURED_WITH)",
                     "bytes_per_launch": dom_bytes, "avg_kernel_us": round(dom_ms * 1e3, 3),
                     # the same call launched back to back, two events around the burst (all of the
                     # call's kernels and the gaps between launches, no per-launch event)
                     "back_to_back_us_per_call": round(b2b * 1e6, 3),
                     "back_to_back_GBps": round(dom_bytes / b2b / 1e9, 1)},
        "kernel_us": {k: round(v[0] * 1e3, 3) for k, v in kt.items()},
        "kernels": headline_roofs,
        "roofline_by_batches_per_launch": by_bpl,
        "single_batch_call": single,
        "per_request_call": per_req,
        "host_engine_batched": host_engine,
        "device_reassembly": reassembly,
        "device_pipeline": pipeline,
        "other_workloads": sweep,
    }
    if not a.no_cpu:
        _log("CPU baseline")
        out["cpu_baseline"] = cpu_baseline(w, a.cpu_seconds)
    print(json.dumps(out))
    ctx.close()
    if ctx_tx is not None:
        ctx_tx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
