"""The receive -> gather -> scatter pipeline with its bookkeeping on the device:
requests that straddle bursts (the reference's rr_cache across rr_recv_ng
bursts, src/transport/dpdk_transport_ng.h:176-218), counts that never visit
the host, application slot states published by the device
(src/splitrpc_server/p2p_rpc_dpdk_server.cc:130,175), and the whole step
recorded into one HIP graph."""
import dataclasses

import numpy as np
import pytest
import torch

import oracle
from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, RingRef, SgContext, SgError, to_dev

from helpers import first_diff

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FREE, RX, WORK = capi.SLOT_FREE, capi.SLOT_RX_COMPLETE, capi.SLOT_WORK_COMPLETE


class Tables:
    """Output tables of the device reassembly, sized for the context."""

    def __init__(self, max_reqs, max_frames):
        self.fs = torch.zeros(max_frames, dtype=torch.int32, device=DEV)
        self.fl = torch.zeros(max_frames, dtype=torch.int32, device=DEV)
        self.rf = torch.zeros(max_reqs + 1, dtype=torch.int32, device=DEV)
        self.tok = torch.zeros(max_reqs, dtype=torch.int64, device=DEV)
        self.hdr = torch.zeros(max_reqs, dtype=torch.int32, device=DEV)
        self.counts = torch.zeros(4, dtype=torch.int32, device=DEV)

    def take(self, n_req, n_frag):
        u32 = lambda t: t.cpu().numpy().view(np.uint32)
        return (u32(self.fs[:n_frag]), u32(self.fl[:n_frag]), u32(self.rf[:n_req + 1]),
                self.tok[:n_req].cpu().numpy().view(np.uint64), u32(self.hdr[:n_req]))


def _feed_in_bursts(ctx, w, order, burst, tabs, len_nic=None, req_size=0, flags=0):
    rx = RingRef(torch.from_numpy(w.ring).to(DEV), w.n_slots, w.slot_size, w.profile)
    arr = to_dev(np.ascontiguousarray(order, np.uint32), DEV)
    ln = to_dev(len_nic, DEV) if len_nic is not None else None
    fs, fl, first, tok, hdr = [], [], [0], [], []
    peak = 0
    b = -1
    nxt = 0
    while nxt < len(order):
        # `burst`: one size for all calls, or a function that says how many arrivals the next call brings
        b, n = nxt, min(burst() if callable(burst) else burst, len(order) - nxt)
        nxt += n
        n_req, n_frag, in_flight = ctx.reassemble(rx, arr[b:b + n], n, tabs.fs, tabs.fl, tabs.rf, tabs.tok,
                                                  ln, req_size, req_hdr_slot=tabs.hdr, counts_out=tabs.counts,
                                                  flags=flags)
        assert tabs.counts.cpu().tolist() == [n_req, n_frag, ctx.last_dropped, in_flight]
        peak = max(peak, in_flight)
        s, l, f, t, h = tabs.take(n_req, n_frag)
        assert f[0] == 0 and f[-1] == n_frag
        fs.append(s), fl.append(l), tok.append(t), hdr.append(h)
        first.extend(int(x) + first[-1] for x in np.diff(f.astype(np.int64)))
    assert in_flight == 0
    return np.concatenate(fs), np.concatenate(fl), np.array(first, np.uint32), np.concatenate(tok), \
        np.concatenate(hdr), peak


@pytest.mark.parametrize("order_kind", ["as generated", "shuffled across requests"])
def test_resnet_sized_requests_arrive_in_bursts_of_64(order_kind):
    """Config 2 at full size, 64 arrivals per call as a NIC burst brings them:
    every 431-fragment request straddles many calls; the calls' outputs laid end
    to end are what the oracle makes of the whole stream."""
    w = synth.make_workload(2)
    order = w.arrivals if order_kind == "as generated" else np.random.default_rng(3).permutation(w.arrivals)
    print(f"case bursts cfg=2 arrivals={len(order)} order={order_kind}", flush=True)
    ctx = SgContext(0, max_reqs=64, max_frames=8192)
    ctx.reassemble_reset()
    tabs = Tables(64, 8192)
    fs, fl, first, tok, hdr, peak = _feed_in_bursts(ctx, w, order, 64, tabs)
    efs, efl, erf, etok = oracle.reassemble(w, arrivals=order)
    assert np.array_equal(tok, etok)
    assert np.array_equal(first, erf)
    assert np.array_equal(fs, efs)
    assert np.array_equal(fl, efl)
    assert np.array_equal(hdr, efs[erf[:-1]])
    assert peak >= (1 if order_kind == "as generated" else w.n_req)
    ctx.close()


@pytest.mark.parametrize("flags", [0, capi.F_SMALL_GROUPS], ids=["groups-of-1024", "groups-of-256"])
@pytest.mark.parametrize("burst", [1000, 1024, 1025, 2500])
def test_bursts_around_the_size_one_workgroup_takes(burst, flags):
    """A burst of up to 1024 arrivals is sorted by one workgroup in one launch,
    a larger one by four kernels (of 1024-thread workgroups, or of 256-thread
    ones as for a call that runs beside a long kernel): the same stream in
    bursts on either side of that size (requests carried across calls both
    ways) gives what the oracle makes of the whole stream."""
    w = synth.make_workload(4, 700)
    order = np.random.default_rng(burst).permutation(w.arrivals)
    ctx = SgContext(0, max_reqs=1024, max_frames=8192)
    ctx.reassemble_reset()
    tabs = Tables(1024, 8192)
    fs, fl, first, tok, hdr, peak = _feed_in_bursts(ctx, w, order, burst, tabs, flags=flags)
    efs, efl, erf, etok = oracle.reassemble(w, arrivals=order)
    assert np.array_equal(tok, etok) and np.array_equal(first, erf)
    assert np.array_equal(fs, efs) and np.array_equal(fl, efl)
    assert np.array_equal(hdr, efs[erf[:-1]])
    assert peak > 10
    ctx.close()


@pytest.mark.parametrize("seed", range(24))
def test_random_streams_in_bursts_of_random_sizes(seed):
    """Seeded random streams -- request sizes, MTU, header profile, arrival order -- cut into calls of
    random sizes on both sides of what one workgroup takes, so that the one-launch and the four-kernel
    form alternate over the same table with requests carried from one to the other."""
    rng = np.random.default_rng(7000 + seed)
    profile = int(rng.integers(0, 2))
    mtu = int(rng.choice([64, 256, 1400]))
    n_req = int(rng.integers(1, 400))
    if profile == synth.HDR_REF64:
        sizes = [int(rng.integers(1, 12 * mtu))] * n_req   # ready when the bytes add up to the one size
    else:
        sizes = [int(x) for x in rng.integers(1, 12 * mtu, n_req)]
    w = synth.make_custom(sizes, [1] * n_req, mtu=mtu, slot_size=2 * ((synth.hdr_len(profile) + mtu + 1) // 2),
                          order=str(rng.choice(["in_order", "perm_within_request", "interleave_keep_order", "shuffle_all"])),
                          seed=seed, profile=profile)
    order = w.arrivals if rng.integers(0, 2) else rng.permutation(w.arrivals)
    menu = [1, 7, 64, 500, 1024, 1025, 3000]
    print(f"case random bursts seed={seed} profile={profile} mtu={mtu} n_req={n_req} arrivals={len(order)}", flush=True)
    ctx = SgContext(0, max_reqs=512, max_frames=8192)
    ctx.reassemble_reset()
    tabs = Tables(512, 8192)
    ln = None
    if profile == synth.HDR_REF64:
        ln = np.zeros(w.n_slots, np.uint32)
        ln[w.frag_slot] = w.frag_len
    fs, fl, first, tok, hdr, _ = _feed_in_bursts(ctx, w, order, lambda: int(rng.choice(menu)), tabs, len_nic=ln,
                                                 req_size=sizes[0] if profile == synth.HDR_REF64 else 0)
    efs, efl, erf, etok = oracle.reassemble(w, arrivals=order, frag_len_nic=ln,
                                            req_size=sizes[0] if profile == synth.HDR_REF64 else 0)
    assert np.array_equal(tok, etok) and np.array_equal(first, erf)
    assert np.array_equal(fs, efs) and np.array_equal(fl, efl)
    assert np.array_equal(hdr, efs[erf[:-1]])
    ctx.close()


def test_bursts_with_the_reference_header_and_nic_lengths():
    """REF64: a request is complete when its bytes add up to the server-wide
    size; the running total is carried from call to call."""
    w = synth.make_workload(1, 20, profile=synth.HDR_REF64)
    len_nic = np.zeros(w.n_slots, np.uint32)
    len_nic[w.frag_slot] = w.frag_len
    order = np.random.default_rng(8).permutation(w.arrivals)
    ctx = SgContext(0, max_reqs=32, max_frames=256)
    tabs = Tables(32, 256)
    size = int(w.req_sizes[0])
    fs, fl, first, tok, hdr, peak = _feed_in_bursts(ctx, w, order, 7, tabs, len_nic=len_nic, req_size=size)
    efs, efl, erf, etok = oracle.reassemble(w, arrivals=order, req_size=size, frag_len_nic=len_nic)
    assert np.array_equal(tok, etok) and np.array_equal(first, erf)
    assert np.array_equal(fs, efs) and np.array_equal(fl, efl)
    assert peak > 3
    ctx.close()


def test_pool_exhaustion_eviction_and_reset():
    """More requests in flight than the pool has records: refused, the rest
    goes on.  Eviction clears out what has been idle; afterwards the table is
    as good as new."""
    w = synth.make_custom([4200] * 9, [64] * 9, seed=41)
    ctx = SgContext(0, max_reqs=4, max_frames=64)
    tabs = Tables(4, 64)
    rx = RingRef(torch.from_numpy(w.ring).to(DEV), w.n_slots, w.slot_size, w.profile)
    firsts = np.ascontiguousarray(w.frag_slot[w.req_first[:6]], np.uint32)  # fragment 0 of six requests
    with pytest.raises(SgError) as e:
        ctx.reassemble(rx, to_dev(firsts, DEV), 6, tabs.fs, tabs.fl, tabs.rf, tabs.tok)
    assert e.value.code == capi.SG_E_DATA and "in flight" in str(e.value)
    # nothing idle yet at age 5; everything parked goes at age 0
    assert ctx.reassemble_evict(5) == 0
    assert ctx.reassemble_evict(0) == 6
    n_req, n_frag, in_flight = ctx.reassemble(rx, to_dev(w.arrivals[:1], DEV), 0, tabs.fs, tabs.fl, tabs.rf, tabs.tok)
    assert (n_req, n_frag, in_flight) == (0, 0, 0)
    # four requests at a time fit
    for lo in (0, 4):
        sel = np.concatenate([w.frag_slot[w.req_first[r]:w.req_first[r + 1]] for r in range(lo, min(lo + 4, 9))])
        n_req, n_frag, in_flight = ctx.reassemble(rx, to_dev(sel.astype(np.uint32), DEV), len(sel), tabs.fs, tabs.fl,
                                                  tabs.rf, tabs.tok)
        assert (n_req, n_frag, in_flight) == (4, 12, 0)
        assert np.array_equal(tabs.take(n_req, n_frag)[0], sel)
    # a parked request, then a reset
    ctx.reassemble(rx, to_dev(firsts[:2], DEV), 2, tabs.fs, tabs.fl, tabs.rf, tabs.tok)
    ctx.reassemble_reset()
    n_req, n_frag, in_flight = ctx.reassemble(rx, to_dev(firsts[:1], DEV), 0, tabs.fs, tabs.fl, tabs.rf, tabs.tok)
    assert in_flight == 0
    ctx.close()


def _sub(w, fs, fl, rf, resp_rows, tx_slots, hdr_slots, resp_size):
    """A workload holding just the requests of one call, for the oracle."""
    n = len(rf) - 1
    per = synth.num_frames(resp_size, w.mtu)
    return dataclasses.replace(
        w, frag_slot=fs, frag_len=fl, req_first=rf.astype(np.uint32),
        req_sizes=np.full(n, int(w.req_sizes[0]), np.uint64), resp_sizes=np.full(n, resp_size, np.uint64),
        resp_first=(np.arange(n + 1) * per).astype(np.uint32), tx_slot=tx_slots[:n * per].astype(np.uint32),
        hdr_src_slot=np.repeat(hdr_slots, per).astype(np.uint32), resp_payload=resp_rows, req_ids=np.zeros(n, np.uint64))


def test_slot_states_published_by_the_device():
    """gather: FREE -> RX_COMPLETE for the slots it filled; scatter: WORK_COMPLETE
    -> FREE; both indices advance on the device and wrap; a slot in the wrong
    state is reported."""
    w = synth.make_custom([4200] * 5, [3000] * 5, seed=51, flags=synth.F_UDP_CSUM_PSEUDO)
    dw = DeviceWorkload(w)
    ctx = SgContext(0)
    n_states = 7
    states = torch.zeros(n_states, dtype=torch.int32, device=DEV)
    ctx.set_slot_index(0, 5)
    ctx.set_slot_index(1, 5)
    for mode in ("rule", "scan"):
        ga = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app, dw.req_offsets,
                             flags=capi.F_RULE_FRAGS if mode == "rule" else 0,
                             fixed_req_size=4200 if mode == "rule" else 0, mtu=w.mtu, slot_state=states)
        pi = ctx.get_slot_index(0)
        ctx.gather_batch_raw(ga)
        want = np.zeros(n_states, np.int32)
        want[(pi + np.arange(5)) % n_states] = RX
        assert np.array_equal(states.cpu().numpy(), want), mode
        assert ctx.get_slot_index(0) == (pi + 5) % n_states
        # the TX side finds them not yet worked on: reported, and (as documented) freed all the same
        sa = ctx.scatter_args(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first,
                              None if mode == "rule" else dw.resp_size, 3000 if mode == "rule" else 0, dw.n_req,
                              dw.n_frames, w.mtu, dw.resp_app, dw.resp_offsets, w.flags, slot_state=states)
        if mode == "rule":
            with pytest.raises(SgError) as e:
                ctx.scatter_batch_raw(sa)
            assert e.value.code == capi.SG_E_DATA and "slot" in str(e.value)
            assert not states.cpu().numpy().any()
            ctx.set_slot_index(1, pi)
            states.copy_(torch.from_numpy(want))
        states[states == RX] = WORK  # the worker
        ctx.scatter_batch_raw(sa)
        assert not states.cpu().numpy().any(), mode
        assert ctx.get_slot_index(1) == (pi + 5) % n_states
    # a refused descriptor-pass batch publishes nothing and advances nothing
    bad = w.frag_slot.copy()
    bad[2] = w.n_slots + 1
    bad_dev = to_dev(bad, DEV)
    ga = ctx.gather_args(dw.rx, bad_dev, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app, dw.req_offsets,
                         slot_state=states)
    pi = ctx.get_slot_index(0)
    with pytest.raises(SgError):
        ctx.gather_batch_raw(ga)
    assert not states.cpu().numpy().any()
    assert ctx.get_slot_index(0) == pi
    # the same bad fragment with the rule declared: the other fragments move and the cursor moves (no
    # descriptor pass has looked at the batch beforehand), but no slot is published -- a worker that
    # polls the words is never handed a request with a hole in it -- and the ring index stays
    ga = ctx.gather_args(dw.rx, bad_dev, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app, dw.req_offsets,
                         flags=capi.F_RULE_FRAGS, fixed_req_size=4200, mtu=w.mtu, slot_state=states)
    c0 = ctx.get_cursor(0)
    with pytest.raises(SgError) as e:
        ctx.gather_batch_raw(ga)
    assert e.value.code == capi.SG_E_DATA
    assert not states.cpu().numpy().any()
    assert ctx.get_slot_index(0) == pi
    assert ctx.get_cursor(0) == (c0 + 5 * 4200) % dw.req_app.cap
    # and on the TX side: a bad TX slot index with one response size
    states.fill_(WORK)
    bad_tx = w.tx_slot.copy()
    bad_tx[1] = w.tx_n_slots + 4
    bad_tx_dev = to_dev(bad_tx, DEV)
    sa = ctx.scatter_args(dw.rx, dw.tx, bad_tx_dev, dw.hdr_src_slot, dw.resp_first, None, 3000, dw.n_req,
                          dw.n_frames, w.mtu, dw.resp_app, dw.resp_offsets, w.flags, slot_state=states)
    ci = ctx.get_slot_index(1)
    with pytest.raises(SgError) as e:
        ctx.scatter_batch_raw(sa)
    assert e.value.code == capi.SG_E_DATA
    assert bool((states == WORK).all())
    assert ctx.get_slot_index(1) == ci
    states.zero_()
    # more requests than the ring has slots: refused by the host
    small = torch.zeros(3, dtype=torch.int32, device=DEV)
    ga = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app, slot_state=small)
    with pytest.raises(SgError) as e:
        ctx.gather_batch_raw(ga)
    assert e.value.code == capi.SG_E_INVAL
    ctx.close()


@pytest.mark.parametrize("use_graph", [False, True], ids=["eager", "one-graph"])
def test_bursts_through_reassembly_gather_and_scatter_without_the_host(use_graph):
    """One step = reassemble + gather + scatter, three calls, none of which
    waits for the host: the counts go from call to call in device memory.  With
    use_graph the three calls (an odd number per arena) are recorded ONCE and
    replayed for every burst; the burst's arrivals and their number are written
    into device buffers between replays.  Every step is held against the oracle:
    request arena, TX ring, bump-ring cursors, slot indices and slot states."""
    n_reqs, burst, resp_size, n_states = 24, 16, 3000, 17
    w = synth.make_custom([4200] * n_reqs, [resp_size] * n_reqs, seed=61,
                          flags=synth.F_UDP_CSUM_PSEUDO | synth.F_IPV4_CSUM)
    order = np.random.default_rng(4).permutation(w.arrivals)
    efs, efl, erf, etok = oracle.reassemble(w, arrivals=order)
    slot_req = {int(s): r for r in range(n_reqs) for s in efs[erf[r]:erf[r + 1]]}
    per_req, per_resp = 3, synth.num_frames(resp_size, w.mtu)
    s = torch.cuda.Stream()
    ctx = SgContext(0, max_reqs=64, max_frames=4096, stream=s.cuda_stream)
    ctx.reassemble_reset()
    tabs = Tables(64, 4096)
    rx_ring = torch.from_numpy(w.ring).to(DEV)
    rx = RingRef(rx_ring, w.n_slots, w.slot_size, w.profile)
    tx_slots = np.random.default_rng(5).permutation(burst * per_resp).astype(np.uint32)
    tx_init = np.random.default_rng(6).integers(0, 256, burst * per_resp * w.slot_size, dtype=np.uint8)
    tx_ring = torch.from_numpy(tx_init).to(DEV)
    tx = RingRef(tx_ring, burst * per_resp, w.slot_size, w.profile)
    req_cap, resp_cap = 17 * 4200 + 100, 7 * resp_size + 50  # the request arena holds a whole burst's worth
    req_arena = torch.zeros(req_cap, dtype=torch.uint8, device=DEV)
    resp_np = np.random.default_rng(7).integers(0, 256, resp_cap, dtype=np.uint8)
    resp_arena = torch.from_numpy(resp_np).to(DEV)
    states = torch.zeros(n_states, dtype=torch.int32, device=DEV)
    arr_buf = torch.zeros(burst, dtype=torch.int32, device=DEV)
    n_arr = torch.zeros(1, dtype=torch.int32, device=DEV)
    tx_slot_dev = to_dev(tx_slots, DEV)
    resp_first = to_dev((np.arange(burst + 1) * per_resp).astype(np.uint32), DEV)

    A = capi.F_ASYNC
    ra = ctx.reassemble_args(rx, arr_buf, burst, tabs.fs, tabs.fl, tabs.rf, tabs.tok, req_hdr_slot=tabs.hdr,
                             counts_out=tabs.counts, n_arrivals_dev=n_arr, flags=A)
    ga = ctx.gather_args(rx, tabs.fs, None, tabs.rf, burst, burst * per_req, AppRef(arena=req_arena, cap=req_cap),
                         None, flags=A | capi.F_RULE_FRAGS, fixed_req_size=4200, mtu=w.mtu, counts=tabs.counts,
                         slot_state=states)
    sa = ctx.scatter_args(rx, tx, tx_slot_dev, None, resp_first, None, resp_size, burst, burst * per_resp, w.mtu,
                          AppRef(arena=resp_arena, cap=resp_cap), None, w.flags | A, hdr_src_req=tabs.hdr,
                          counts=tabs.counts, slot_state=states)

    def step():
        ctx.reassemble_raw(ra)
        ctx.gather_batch_raw(ga)
        with torch.cuda.stream(s):
            states.copy_(torch.where(states == RX, torch.full_like(states, WORK), states))  # the worker
        ctx.scatter_batch_raw(sa)

    ctx.set_cursor(0, req_cap - 5000)
    ctx.set_cursor(1, 0)
    ctx.set_slot_index(0, n_states - 3)
    ctx.set_slot_index(1, n_states - 3)
    torch.cuda.synchronize()
    g = None
    if use_graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            step()
    want_req = np.zeros(req_cap, np.uint8)
    want_tx = tx_init.copy()
    cur0, cur1, done, idx = req_cap - 5000, 0, 0, n_states - 3
    pos_done = np.zeros(n_reqs, int)  # fragments seen per request (in completion-order numbering)
    for b in range(0, len(order), burst):
        part = order[b:b + burst]
        arr_buf[:len(part)] = to_dev(np.ascontiguousarray(part, np.uint32), DEV)
        n_arr.fill_(len(part))
        torch.cuda.synchronize()
        if use_graph:
            g.replay()
        else:
            step()
        torch.cuda.synchronize()
        ctx.sync()
        for sl in part:
            pos_done[slot_req[int(sl)]] += 1
        now = int((pos_done == per_req).sum())
        r0, r1 = done, now
        counts = tabs.counts.cpu().tolist()
        assert counts[:2] == [r1 - r0, (r1 - r0) * per_req], f"burst at {b}: {counts}"
        assert counts[3] == int(((pos_done > 0) & (pos_done < per_req)).sum())
        if r1 > r0:
            fs = efs[erf[r0]:erf[r1]]
            sub = _sub(w, fs, efl[erf[r0]:erf[r1]], erf[r0:r1 + 1] - erf[r0], None, tx_slots, efs[erf[r0:r1]],
                       resp_size)
            want_req, _, cur0 = oracle.gather(sub, arena_cap=req_cap, cursor=cur0, out=want_req)
            sub.tx_n_slots = burst * per_resp
            _, cur1 = oracle.scatter(sub, w.ring, want_tx, resp_np, arena_cap=resp_cap, cursor=cur1)
        done = now
        idx = (idx + (r1 - r0)) % n_states
        got = req_arena.cpu().numpy()
        assert np.array_equal(got, want_req), f"burst at {b}: " + first_diff(got, want_req)
        got = tx_ring.cpu().numpy()
        assert np.array_equal(got, want_tx), f"burst at {b}: " + first_diff(got, want_tx)
        assert ctx.get_cursor(0) == cur0 and ctx.get_cursor(1) == cur1
        assert ctx.get_slot_index(0) == idx and ctx.get_slot_index(1) == idx
        assert not states.cpu().numpy().any()
    assert done == n_reqs
    ctx.close()


@pytest.mark.parametrize("burst", [7, 16, 40])
def test_reassembly_on_a_stream_of_its_own_beside_the_copy(burst):
    """The receive path with burst k + 1 being filed while burst k is gathered
    and answered: the reassembly on one context (stream), gather + scatter
    (sg_hip_shunt_batch) on another, the reassembly's output tables
    double-buffered and events between the two streams -- every burst queued,
    the host waiting for nothing until the end.  Final request arena, TX ring
    and cursors against the oracle's reassembly, gather and scatter replayed
    burst by burst."""
    n_reqs, resp_size = 36, 3000
    w = synth.make_custom([4200] * n_reqs, [resp_size] * n_reqs, seed=63,
                          flags=synth.F_UDP_CSUM_PSEUDO | synth.F_IPV4_CSUM)
    order = np.random.default_rng(14).permutation(w.arrivals)
    efs, efl, erf, etok = oracle.reassemble(w, arrivals=order)
    slot_req = {int(s): r for r in range(n_reqs) for s in efs[erf[r]:erf[r + 1]]}
    per_req, per_resp = 3, synth.num_frames(resp_size, w.mtu)
    ctx_ra = SgContext(0, max_reqs=64, max_frames=4096)
    ctx_sg = SgContext(0, max_reqs=64, max_frames=4096)
    ctx_ra.reassemble_reset()
    s_ra = torch.cuda.ExternalStream(ctx_ra.stream, device=DEV)
    s_sg = torch.cuda.ExternalStream(ctx_sg.stream, device=DEV)
    sets = [Tables(64, 4096), Tables(64, 4096)]
    rx = RingRef(torch.from_numpy(w.ring).to(DEV), w.n_slots, w.slot_size, w.profile)
    bound = min(burst, n_reqs)  # a burst of b arrivals completes at most b requests
    tx_slots = np.random.default_rng(15).permutation(bound * per_resp).astype(np.uint32)
    tx_init = np.random.default_rng(16).integers(0, 256, bound * per_resp * w.slot_size, dtype=np.uint8)
    tx_ring = torch.from_numpy(tx_init).to(DEV)
    tx = RingRef(tx_ring, bound * per_resp, w.slot_size, w.profile)
    req_cap, resp_cap = n_reqs * 4200 + 100, 7 * resp_size + 50  # every request of the run keeps its place
    req_arena = torch.zeros(req_cap, dtype=torch.uint8, device=DEV)
    resp_np = np.random.default_rng(17).integers(0, 256, resp_cap, dtype=np.uint8)
    resp_arena = torch.from_numpy(resp_np).to(DEV)
    arr = to_dev(np.ascontiguousarray(order, np.uint32), DEV)
    tx_slot_dev = to_dev(tx_slots, DEV)
    resp_first = to_dev((np.arange(bound + 1) * per_resp).astype(np.uint32), DEV)
    A = capi.F_ASYNC
    gas, sas = [], []
    for t in sets:
        gas.append(ctx_sg.gather_args(rx, t.fs, None, t.rf, bound, bound * per_req, AppRef(arena=req_arena, cap=req_cap),
                                      None, flags=A | capi.F_RULE_FRAGS, fixed_req_size=4200, mtu=w.mtu,
                                      counts=t.counts))
        sas.append(ctx_sg.scatter_args(rx, tx, tx_slot_dev, None, resp_first, None, resp_size, bound,
                                       bound * per_resp, w.mtu, AppRef(arena=resp_arena, cap=resp_cap), None,
                                       w.flags | A, hdr_src_req=t.hdr, counts=t.counts))
    start = req_cap - 5000
    ctx_sg.set_cursor(0, start)
    ctx_sg.set_cursor(1, 0)
    torch.cuda.synchronize()
    filled = [torch.cuda.Event(), torch.cuda.Event()]
    drained = [None, None]
    keep = []
    for k, b in enumerate(range(0, len(order), burst)):
        j = k & 1
        t = sets[j]
        n = min(burst, len(order) - b)
        if drained[j] is not None:
            s_ra.wait_event(drained[j])          # the copy of burst k - 2 has read this set
        ra = ctx_ra.reassemble_args(rx, arr[b:b + n], n, t.fs, t.fl, t.rf, t.tok, req_hdr_slot=t.hdr,
                                    counts_out=t.counts, flags=A)
        keep.append(ra)
        ctx_ra.reassemble_raw(ra)
        filled[j].record(s_ra)
        s_sg.wait_event(filled[j])               # the copy of burst k starts once its tables are in
        ctx_sg.shunt_batch_raw(gas[j], sas[j])
        drained[j] = torch.cuda.Event()
        drained[j].record(s_sg)
    ctx_ra.sync()
    ctx_sg.sync()
    torch.cuda.synchronize()
    # the oracle, burst by burst
    want_req = np.zeros(req_cap, np.uint8)
    want_tx = tx_init.copy()
    cur0, cur1, done = start, 0, 0
    pos_done = np.zeros(n_reqs, int)
    for b in range(0, len(order), burst):
        for sl in order[b:b + burst]:
            pos_done[slot_req[int(sl)]] += 1
        now = int((pos_done == per_req).sum())
        r0, r1 = done, now
        if r1 > r0:
            sub = _sub(w, efs[erf[r0]:erf[r1]], efl[erf[r0]:erf[r1]], erf[r0:r1 + 1] - erf[r0], None, tx_slots,
                       efs[erf[r0:r1]], resp_size)
            want_req, _, cur0 = oracle.gather(sub, arena_cap=req_cap, cursor=cur0, out=want_req)
            sub.tx_n_slots = bound * per_resp
            _, cur1 = oracle.scatter(sub, w.ring, want_tx, resp_np, arena_cap=resp_cap, cursor=cur1)
        done = now
    assert done == n_reqs
    got = req_arena.cpu().numpy()
    assert np.array_equal(got, want_req), first_diff(got, want_req)
    got = tx_ring.cpu().numpy()
    assert np.array_equal(got, want_tx), first_diff(got, want_tx)
    assert ctx_sg.get_cursor(0) == cur0 and ctx_sg.get_cursor(1) == cur1
    ctx_ra.close()
    ctx_sg.close()


@pytest.mark.parametrize("threaded", [0, 1])
def test_receive_queues_side_by_side_from_a_native_loop(threaded):
    """Three receive queues, each with a context (stream, reassembly table,
    cursors), rings and tables of its own, every queue's bursts filed,
    gathered and answered from a native loop with no host wait
    (sgh_pipeline_queues_gpu of libsg_host.so, from one thread or from a
    thread per queue): each queue's request arena,
    TX ring and cursors against the oracle's reassembly, gather and scatter
    replayed burst by burst."""
    import ctypes as C
    from splitrpc_amd import build
    host = C.CDLL(build.HOST_LIB)
    host.sgh_pipeline_queues_gpu.restype = C.c_double
    host.sgh_pipeline_queues_gpu.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                             C.c_int]
    n_queues, burst, n_reqs, resp_size = 3, 16, 30, 3000
    per_req, A = 3, capi.F_ASYNC
    queues = []
    for q in range(n_queues):
        w = synth.make_custom([4200] * n_reqs, [resp_size] * n_reqs, seed=70 + q,
                              flags=synth.F_UDP_CSUM_PSEUDO | synth.F_IPV4_CSUM)
        order = np.random.default_rng(20 + q).permutation(w.arrivals)
        per_resp = synth.num_frames(resp_size, w.mtu)
        ctx = SgContext(0, max_reqs=64, max_frames=4096)
        ctx.reassemble_reset()
        t = Tables(64, 4096)
        rx = RingRef(torch.from_numpy(w.ring).to(DEV), w.n_slots, w.slot_size, w.profile)
        bound = min(burst, n_reqs)
        tx_slots = np.random.default_rng(30 + q).permutation(bound * per_resp).astype(np.uint32)
        tx_init = np.random.default_rng(40 + q).integers(0, 256, bound * per_resp * w.slot_size, dtype=np.uint8)
        tx_ring = torch.from_numpy(tx_init).to(DEV)
        tx = RingRef(tx_ring, bound * per_resp, w.slot_size, w.profile)
        req_cap, resp_cap = n_reqs * 4200 + 100 + q, 7 * resp_size + 50
        req_arena = torch.zeros(req_cap, dtype=torch.uint8, device=DEV)
        resp_np = np.random.default_rng(50 + q).integers(0, 256, resp_cap, dtype=np.uint8)
        resp_arena = torch.from_numpy(resp_np).to(DEV)
        arr = to_dev(np.ascontiguousarray(order, np.uint32), DEV)
        tx_slot_dev = to_dev(tx_slots, DEV)
        resp_first = to_dev((np.arange(bound + 1) * per_resp).astype(np.uint32), DEV)
        ga = ctx.gather_args(rx, t.fs, None, t.rf, bound, bound * per_req, AppRef(arena=req_arena, cap=req_cap), None,
                             flags=A | capi.F_RULE_FRAGS, fixed_req_size=4200, mtu=w.mtu, counts=t.counts)
        sa = ctx.scatter_args(rx, tx, tx_slot_dev, None, resp_first, None, resp_size, bound, bound * per_resp, w.mtu,
                              AppRef(arena=resp_arena, cap=resp_cap), None, w.flags | A, hdr_src_req=t.hdr,
                              counts=t.counts)
        ras = [ctx.reassemble_args(rx, arr[b:b + burst], min(burst, len(order) - b), t.fs, t.fl, t.rf, t.tok,
                                   req_hdr_slot=t.hdr, counts_out=t.counts, flags=A)
               for b in range(0, len(order), burst)]
        start = req_cap - 5000 - 100 * q
        ctx.set_cursor(0, start)
        ctx.set_cursor(1, 0)
        queues.append(dict(w=w, order=order, ctx=ctx, t=t, rx=rx, tx_slots=tx_slots, tx_init=tx_init, tx_ring=tx_ring,
                           tx=tx, req_cap=req_cap, resp_cap=resp_cap, req_arena=req_arena, resp_np=resp_np,
                           resp_arena=resp_arena, arr=arr, keep=(tx_slot_dev, resp_first), ga=ga, sa=sa, ras=ras,
                           start=start, bound=bound, per_resp=per_resp))
    n_bursts = len(queues[0]["ras"])
    assert all(len(q["ras"]) == n_bursts for q in queues)
    ptrs = lambda xs: (C.c_void_p * len(xs))(*[C.addressof(x) for x in xs])
    c_ctx = (C.c_void_p * n_queues)(*[q["ctx"].h for q in queues])
    c_ras = ptrs([ra for q in queues for ra in q["ras"]])
    c_ga = ptrs([q["ga"] for q in queues for _ in range(n_bursts)])
    c_sa = ptrs([q["sa"] for q in queues for _ in range(n_bursts)])
    torch.cuda.synchronize()
    print(f"case queues={n_queues} bursts={n_bursts} of {burst} threaded={threaded}", flush=True)
    dt = host.sgh_pipeline_queues_gpu(c_ctx, n_queues, c_ras, c_ga, c_sa, n_bursts, threaded)
    assert dt > 0, (dt, [q["ctx"].lib.sg_hip_last_error(q["ctx"].h) for q in queues])
    torch.cuda.synchronize()
    for qi, q in enumerate(queues):
        w, order = q["w"], q["order"]
        efs, efl, erf, _ = oracle.reassemble(w, arrivals=order)
        slot_req = {int(s): r for r in range(n_reqs) for s in efs[erf[r]:erf[r + 1]]}
        want_req = np.zeros(q["req_cap"], np.uint8)
        want_tx = q["tx_init"].copy()
        cur0, cur1, done = q["start"], 0, 0
        pos_done = np.zeros(n_reqs, int)
        for b in range(0, len(order), burst):
            for sl in order[b:b + burst]:
                pos_done[slot_req[int(sl)]] += 1
            now = int((pos_done == per_req).sum())
            if now > done:
                r0, r1 = done, now
                sub = _sub(w, efs[erf[r0]:erf[r1]], efl[erf[r0]:erf[r1]], erf[r0:r1 + 1] - erf[r0], None,
                           q["tx_slots"], efs[erf[r0:r1]], resp_size)
                want_req, _, cur0 = oracle.gather(sub, arena_cap=q["req_cap"], cursor=cur0, out=want_req)
                sub.tx_n_slots = q["bound"] * q["per_resp"]
                _, cur1 = oracle.scatter(sub, w.ring, want_tx, q["resp_np"], arena_cap=q["resp_cap"], cursor=cur1)
            done = now
        assert done == n_reqs
        got = q["req_arena"].cpu().numpy()
        assert np.array_equal(got, want_req), (qi, first_diff(got, want_req))
        got = q["tx_ring"].cpu().numpy()
        assert np.array_equal(got, want_tx), (qi, first_diff(got, want_tx))
        assert q["ctx"].get_cursor(0) == cur0 and q["ctx"].get_cursor(1) == cur1, qi
    for q in queues:
        q["ctx"].close()
