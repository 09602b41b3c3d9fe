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
    (2, 32, "k_gather"): 653.6e6, (2, 32, "k_scatter"): 4.7e6,
    (1, 2048, "k_gather"): 450.5e6, (1, 2048, "k_scatter"): 22.5e6,
    (3, 512, "k_gather"): 585.7e6, (3, 512, "k_scatter"): 934.7e6,
    (4, 8, "k_gather"): 661.9e6, (4, 8, "k_scatter"): 676.0e6,
    (5, 4, "k_gather"): 817.6e6, (5, 4, "k_scatter"): 549.3e6,
}
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


def timed(ctx, pool: Pool, steps: int, warmup: int, ctx_tx=None, reps: int = 5):
    """Seconds per step: `warmup` untimed steps, then `reps` timed runs of
    exactly `steps` steps each, bracketed by synchronization on both sides; the
    median run is reported (one run of 20 steps of 0.1 ms is a 2 ms sample)."""
    import torch
    from splitrpc_amd import capi

    def drain():
        ctx.sync()
        if ctx_tx is not None:
            ctx_tx.sync()
        torch.cuda.synchronize()

    # every rotated copy is touched at least once before the clock starts
    for i in range(max(warmup, len(pool.items))):
        pool.step(ctx, i, capi.F_ASYNC, ctx_tx)
    drain()
    runs = []
    for rep in range(reps):
        t0 = time.perf_counter()
        for i in range(steps):
            pool.step(ctx, warmup + i, capi.F_ASYNC, ctx_tx)
        drain()
        runs.append((time.perf_counter() - t0) / steps)
    runs.sort()
    return runs[len(runs) // 2]


def kernel_times(ctx, pool: Pool, steps: int):
    """Average duration of each kernel from HIP events recorded around every
    launch on the stream the kernels run on."""
    from splitrpc_amd import capi
    ctx.set_profiling(True)
    for i in range(steps):
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
    t0 = time.perf_counter()
    for i in range(calls):
        fn(ctx.h, C.byref(skbs[i % len(skbs)]))
    dt = (time.perf_counter() - t0) / calls
    size = int(w.req_sizes[0])
    return {"us_per_gather_call": round(dt * 1e6, 2), "runs_per_request": int(skbs[0].num_items),
            "request_bytes": size, "requests_per_sec": round(1.0 / dt, 1),
            "GBps": round((2 * size + 16 * int(skbs[0].num_items)) / dt / 1e9, 2)}


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


def graph_step_time(w, extra: int, rule: bool, rotate_mb: int, steps: int = 16, replays: int = 50,
                    streams: int = 1):
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
        stream = torch.cuda.Stream()
        ctx = SgContext(0, max_reqs=max(4096, w.n_req), max_frames=max(65536, w.n_frags, w.n_resp_frames),
                        stream=stream.cuda_stream)
        pool = Pool(w, 1, max(64, rotate_mb // streams), extra, rule=rule)
        for i in range(len(pool.items)):
            pool.step(ctx, i, capi.F_ASYNC)
        ctx.sync()
        lanes.append((stream, ctx, pool))
    torch.cuda.synchronize()
    graphs = []
    for stream, ctx, pool in lanes:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(steps):
                pool.step(ctx, i, capi.F_ASYNC)
        graphs.append(g)

    def replay_all():
        for (stream, _, _), g in zip(lanes, graphs):
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
    for _, ctx, _ in lanes:
        ctx.sync()
        ctx.close()
    return dt


def device_pipeline(w, dw, bursts=(256, 1024, 4096)) -> dict:
    """The receive path end to end on the device, burst after burst and no
    host wait in between: sg_hip_reassemble files a burst's arrivals (requests
    that stay incomplete wait on the device), sg_hip_gather_batch gathers the
    requests the burst completed (their number stays on the device),
    sg_hip_scatter_batch answers them.  All arrivals of one default call's
    worth of requests, in arrival order; wall time over the whole stream."""
    import numpy as np
    import torch
    from splitrpc_amd import capi
    from splitrpc_amd.engine import AppRef, RingRef, SgContext, to_dev
    if w.in_tensor_sizes or w.out_tensor_sizes or w.tx_in_place or len(set(int(x) for x in w.req_sizes)) != 1:
        return None
    dev = "cuda:0"
    size, rsize = int(w.req_sizes[0]), int(w.resp_sizes[0])
    per, per_resp = -(-size // w.mtu), -(-rsize // w.mtu)
    n_arr = int(dw.arrivals.numel())
    out = {"arrivals": n_arr, "requests": dw.n_req}
    for burst in bursts:
        bound = burst // per + 2                      # requests one burst can complete
        ctx = SgContext(0, max_reqs=max(4096, dw.n_req), max_frames=max(65536, bound * per))
        ctx.reassemble_reset()
        i32 = lambda n: torch.zeros(n, dtype=torch.int32, device=dev)
        fs, fl, rf, hdr, counts = i32(max(65536, bound * per)), i32(max(65536, bound * per)), i32(4097 + dw.n_req), \
            i32(4096 + dw.n_req), i32(4)
        req_cap, resp_cap = 4 * bound * size, 4 * bound * rsize
        req_arena = torch.zeros(req_cap, dtype=torch.uint8, device=dev)
        resp_arena = torch.zeros(resp_cap, dtype=torch.uint8, device=dev)
        tx_ring = torch.zeros(bound * per_resp * w.slot_size, dtype=torch.uint8, device=dev)
        tx = RingRef(tx_ring, bound * per_resp, w.slot_size, w.profile)
        tx_slot = to_dev(np.arange(bound * per_resp, dtype=np.uint32), dev)
        resp_first = to_dev((np.arange(bound + 1) * per_resp).astype(np.uint32), dev)
        A = capi.F_ASYNC
        ga = ctx.gather_args(dw.rx, fs, None, rf, bound, bound * per, AppRef(arena=req_arena, cap=req_cap), None,
                             flags=A | capi.F_RULE_FRAGS, fixed_req_size=size, mtu=w.mtu, counts=counts)
        sa = ctx.scatter_args(dw.rx, tx, tx_slot, None, resp_first, None, rsize, bound, bound * per_resp, w.mtu,
                              AppRef(arena=resp_arena, cap=resp_cap), None, w.flags | A, hdr_src_req=hdr, counts=counts)
        ras = [ctx.reassemble_args(dw.rx, dw.arrivals[b:b + burst], min(burst, n_arr - b), fs, fl, rf,
                                   req_hdr_slot=hdr, counts_out=counts, flags=A) for b in range(0, n_arr, burst)]
        torch.cuda.synchronize()
        best = None
        for rep in range(3):
            ctx.reassemble_reset()
            t0 = time.perf_counter()
            for k, ra in enumerate(ras):
                ctx.reassemble_raw(ra)
                ctx.gather_batch_raw(ga)
                ctx.scatter_batch_raw(sa)
                if k % 64 == 63:
                    ctx.sync()
            ctx.sync()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        left = int(counts.cpu()[3])
        out[str(burst)] = {"us_per_burst": round(best / len(ras) * 1e6, 2), "arrivals_per_sec": round(n_arr / best, 1),
                           "requests_per_sec": round(dw.n_req / best, 1),
                           "payload_Gbit_per_sec": round(8.0 * size * dw.n_req / best / 1e9, 1),
                           "requests_left_in_flight": left}
        ctx.close()
        del fs, fl, rf, hdr, counts, req_arena, resp_arena, tx_ring
        torch.cuda.empty_cache()
    return out


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
        # gather and scatter each on a context (and stream) of their own, unless one stream is asked for
        return SgContext(0, max_reqs=mr, max_frames=mf), (None if a.one_stream else SgContext(0, max_reqs=mr, max_frames=mf))

    ctx, ctx_tx = contexts(w, bpl)
    _log(f"staging {w.name} x {bpl} batches per launch")
    pool = Pool(w, bpl, a.rotate_mb, extra, rule=rule)
    _log(f"{len(pool.items)} ring copies staged")

    if a.calib_copy:
        src = torch.empty(512 << 20, dtype=torch.uint8, device="cuda:0").fill_(3)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    sec = timed(ctx, pool, a.steps, a.warmup, ctx_tx)
    _log(f"timed: {sec * 1e6:.1f} us per step (median of 5 runs of {a.steps} steps)")
    kt = kernel_times(ctx, pool, min(a.steps, 100))
    total_bytes = pool.gather_bytes + pool.scatter_bytes
    value = total_bytes / sec / 1e9
    dom = "k_gather" if pool.gather_bytes >= pool.scatter_bytes else "k_scatter"
    dom_bytes = pool.gather_bytes if dom == "k_gather" else pool.scatter_bytes
    dom_ms = kt[dom][0]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9 if dom_ms > 0 else 0.0
    b2b = back_to_back(ctx, pool, dom, min(a.steps, 100))
    # the counters were read with the default kernels and headers only
    traffic_known = not (a.general or a.ref64 or a.no_small or a.no_remap)
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
    t0 = time.perf_counter()
    for b in range(0, n_b, 64):
        ctx.reassemble(dw0.rx, dw0.arrivals[b:b + 64], min(64, n_b - b), ra_fs, ra_fl, ra_rf, **ra_kw)
    reassembly["us_per_burst_of_64"] = round((time.perf_counter() - t0) / max(1, (n_b + 63) // 64) * 1e6, 2)
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
    pipeline = device_pipeline(w, dw0) if not a.ref64 else None

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
    # the single-batch call of the same workload, for the record
    single = None
    if bpl != 1 and not a.no_single:
        p1 = Pool(w, 1, a.rotate_mb, extra, rule=rule)
        s1 = timed(ctx, p1, a.steps, a.warmup, ctx_tx)
        k1 = kernel_times(ctx, p1, min(a.steps, 100))
        b1 = p1.gather_bytes + p1.scatter_bytes
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
        del p1
        for n_streams in (1, 2, 4):
            sg = graph_step_time(w, extra, rule, a.rotate_mb, streams=n_streams)
            key = "hip_graph" if n_streams == 1 else f"hip_graph_{n_streams}_streams"
            single[key + "_ms_per_step"] = round(sg * 1e3, 5)
            single[key + "_GBps"] = round(b1 / sg / 1e9, 1)
            single[key + "_requests_per_sec"] = round(w.n_req / sg, 1)
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
            rps[wc.name] = round(pc.n_req / sc, 1)
            sweep[wc.name] = {"batches_per_launch": b, "ms_per_step": round(sc * 1e3, 5),
                              "GBps": round((pc.gather_bytes + pc.scatter_bytes) / sc / 1e9, 2),
                              "frac_of_hbm_peak": round((pc.gather_bytes + pc.scatter_bytes) / sc / 1e9 / HBM_PEAK_GBS, 4),
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
        sr = timed(ctx, pr, max(20, a.steps // 4), max(5, a.warmup // 4), ctx_tx, reps=3)
        sweep[wr.name + "_ref64_headers"] = {"batches_per_launch": bpl, "ms_per_step": round(sr * 1e3, 5),
                                             "GBps": round((pr.gather_bytes + pr.scatter_bytes) / sr / 1e9, 2)}
        del pr

    out = {
        "metric": "gather+scatter GB/s (algorithmic bytes) on 1 MI355X",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(sec * 1e3, 5),
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
                   "timing": f"median of 5 runs of {a.steps} steps", "flags": w.flags,
                   "tx_slots": "ring order" if a.tx_in_order else "random permutation of the TX ring"},
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "requests_per_sec": rps,
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get((a.workload, bpl, dom)) if traffic_known else None,
                     "traffic_unit": "HBM bytes per launch (rocprofv3 --pmc, see profiles/)",
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
