"""The bump-ring cursors on the device (P2pRpcTring::prev_offset,
src/p2p_rpc_tring.h:14-33): a context's single-kernel calls advance them
themselves, descriptor-path calls and calls that publish slot states through a
kernel behind the copy -- one cursor whatever the order of the calls."""
import numpy as np
import pytest
import torch

import oracle
from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, RingRef, SgContext, to_dev
from helpers import first_diff

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture()
def ctx():
    c = SgContext(0, max_reqs=4096, max_frames=1 << 17)
    yield c
    c.close()


def test_one_cursor_through_calls_of_every_kind(ctx):
    """Declared rule (a small call: the copy kernel advances the cursor), prefix
    scan and declared size (the descriptor pass stages, the copy kernel
    commits), a declared-rule call with a slot ring or with the trailing kernel
    asked for (the kernel behind the copy advances): every call starts where the
    last one ended, on an arena the batch does not divide."""
    sizes = [4200] * 5
    w = synth.make_custom(sizes, [64] * 5, seed=77)
    cap = 3 * sum(sizes) + 1234
    dw = DeviceWorkload(w)
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    app = AppRef(arena=arena, cap=cap)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    states = torch.zeros(64, dtype=torch.int32, device=DEV)
    cur = cap - 9000
    ctx.set_cursor(0, cur)
    ctx.set_slot_index(0, 0)
    want = np.zeros(cap, np.uint8)
    kinds = ["rule", "rule", "scan", "rule", "fixed", "slots", "rule", "tail", "rule", "slots", "scan", "tail", "tail",
             "rule", "rule"]
    for call, kind in enumerate(kinds):
        print(f"case cursor kinds call={call} kind={kind}", flush=True)
        kw = dict(flags=0, fixed_req_size=0, mtu=w.mtu)
        if kind in ("rule", "slots", "tail"):
            kw.update(flags=capi.F_RULE_FRAGS | (capi.F_TAIL_KERNEL if kind == "tail" else 0), fixed_req_size=sizes[0])
        elif kind == "fixed":
            kw.update(fixed_req_size=sizes[0])
        if kind == "slots":
            states.zero_()
            ctx.set_slot_index(0, 0)
            kw.update(slot_state=states)
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs, **kw)
        exp, eoffs, ecur = oracle.gather(w, arena_cap=cap, cursor=cur, out=want)
        got = arena.cpu().numpy()
        assert np.array_equal(got, exp), f"call {call} ({kind}): " + first_diff(got, exp)
        assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs), f"call {call} ({kind})"
        assert ctx.get_cursor(0) == ecur, f"call {call} ({kind})"
        cur = ecur


@pytest.mark.parametrize("form", [capi.F_SELF_ADVANCE, capi.F_TAIL_KERNEL, 0])
def test_queued_calls_of_more_wavefronts_than_the_chip_holds(ctx, form):
    """Four declared-rule gathers queued without a wait between them, each of
    27584 wavefronts.  Where the copy kernel advances the cursor itself
    (forced here: the library keeps that form for smaller calls), most
    wavefronts of a call start long after its first one has written the
    successor, and every one of them still has to take the cursor the call
    began with."""
    w = synth.make_workload(2, 64)
    per_call = int(w.req_sizes.sum())
    calls = 4
    cap = calls * per_call + 4096
    dw = DeviceWorkload(w)
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    app = AppRef(arena=arena, cap=cap)
    offs = [torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV) for _ in range(calls)]
    start = cap - per_call - 777  # the second call wraps
    ctx.set_cursor(0, start)
    torch.cuda.synchronize()
    for k in range(calls):
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs[k],
                         flags=capi.F_RULE_FRAGS | capi.F_ASYNC | form, fixed_req_size=int(w.req_sizes[0]), mtu=w.mtu)
    ctx.sync()
    want = np.zeros(cap, np.uint8)
    cur = start
    for k in range(calls):
        want, eoffs, cur = oracle.gather(w, arena_cap=cap, cursor=cur, out=want)
        assert np.array_equal(offs[k].cpu().numpy().view(np.uint64), eoffs), f"offsets of call {k}"
    assert ctx.get_cursor(0) == cur
    got = arena.cpu().numpy()
    assert np.array_equal(got, want), first_diff(got, want)


@pytest.mark.parametrize("form", [capi.F_SELF_ADVANCE, capi.F_TAIL_KERNEL])
@pytest.mark.parametrize("n_req", [1500, 40])
def test_response_cursor_through_two_kernel_scatters(ctx, n_req, form):
    """Responses of 1400 + 1400 + 272 bytes: with enough of them the remainder
    frames go to a kernel of their own behind the full frames' kernel; both read
    the response cursor and only the second one advances it.  Three calls in a
    row on an arena the batch does not divide, the last two queued."""
    w = synth.make_custom([64] * n_req, [3072] * n_req, seed=78)
    dw = DeviceWorkload(w)
    total = int(w.resp_sizes.sum())
    cap = total + 4000
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    cur = cap - 5000
    ctx.set_cursor(1, cur)
    txs = [to_dev(w.tx_ring_init, DEV) for _ in range(3)]
    exp_tx = []
    for k in range(3):
        # the responses where this call's cursor puts them
        src = np.zeros(cap, np.uint8)
        idx = (cur + np.arange(total, dtype=np.int64)) % cap
        src[idx] = w.resp_payload
        tx = w.tx_ring_init.copy()
        _, ecur = oracle.scatter(w, w.ring, tx, src, arena_cap=cap, cursor=cur)
        exp_tx.append((src, tx, ecur))
        cur = ecur
    arenas = [to_dev(e[0], DEV) for e in exp_tx]
    torch.cuda.synchronize()
    for k in range(3):
        ring = RingRef(txs[k], w.tx_n_slots, w.slot_size, w.profile)
        ctx.scatter_batch(dw.rx, ring, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, None, 3072, w.n_req,
                          w.n_resp_frames, w.mtu, AppRef(arena=arenas[k], cap=cap), offs,
                          w.flags | form | (capi.F_ASYNC if k else 0))
        if k == 0:
            assert ctx.get_cursor(1) == exp_tx[0][2]
    ctx.sync()
    assert ctx.get_cursor(1) == exp_tx[2][2]
    for k in range(3):
        got = txs[k].cpu().numpy()
        assert np.array_equal(got, exp_tx[k][1]), f"call {k}: " + first_diff(got, exp_tx[k][1])


def test_eager_calls_and_graph_replays_in_turns():
    """A recorded call replayed from another stream than the one the context
    launches its eager calls on, the two in turns: launches from different
    queues, one cursor."""
    w = synth.make_workload(1, 8)
    batch = int(w.req_sizes.sum())
    cap = 3 * batch + 1000
    s = torch.cuda.Stream()
    c = SgContext(0, max_reqs=64, max_frames=8192, stream=s.cuda_stream)
    dw = DeviceWorkload(w)
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    app = AppRef(arena=arena, cap=cap)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    a = c.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs,
                      flags=capi.F_ASYNC | capi.F_RULE_FRAGS, fixed_req_size=int(w.req_sizes[0]), mtu=w.mtu)
    c.set_cursor(0, 500)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        c.gather_batch_raw(a)
    want = np.zeros(cap, np.uint8)
    cur = 500
    for rep in range(6):
        print(f"case eager and replay in turns rep={rep}", flush=True)
        for how in ("eager", "replay", "replay", "eager"):
            if how == "eager":
                c.gather_batch_raw(a)
                c.sync()
            else:
                g.replay()
                torch.cuda.synchronize()
            want, eoffs, cur = oracle.gather(w, arena_cap=cap, cursor=cur, out=want)
            assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs), f"{how} in round {rep}"
            assert c.get_cursor(0) == cur
    got = arena.cpu().numpy()
    assert np.array_equal(got, want), first_diff(got, want)
    c.close()


def test_small_and_large_calls_in_turns():
    """A call of more wavefronts than the library picks the self-advancing form
    for leaves the cursor to the kernel behind it; small calls before and after
    it advance it themselves.  One cursor through both."""
    big_w = synth.make_workload(2, 160)   # 68960 wavefronts
    small_w = synth.make_workload(2, 2)
    size = int(big_w.req_sizes[0])
    cap = 170 * size + 999
    big, small = DeviceWorkload(big_w), DeviceWorkload(small_w)
    c = SgContext(0, max_reqs=256, max_frames=1 << 17)
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    app = AppRef(arena=arena, cap=cap)
    offs = torch.zeros(161, dtype=torch.int64, device=DEV)
    cur = cap - 3 * size - 17
    c.set_cursor(0, cur)
    want = np.zeros(cap, np.uint8)
    for call, (w, dw) in enumerate([(small_w, small), (big_w, big), (small_w, small), (small_w, small), (big_w, big),
                                    (small_w, small)]):
        print(f"case small and large calls call={call} n_req={w.n_req}", flush=True)
        c.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs,
                       flags=capi.F_RULE_FRAGS, fixed_req_size=size, mtu=w.mtu)
        want, eoffs, cur = oracle.gather(w, arena_cap=cap, cursor=cur, out=want)
        assert np.array_equal(offs.cpu().numpy().view(np.uint64)[:w.n_req + 1], eoffs), f"call {call}"
        assert c.get_cursor(0) == cur, f"call {call}"
    got = arena.cpu().numpy()
    assert np.array_equal(got, want), first_diff(got, want)
    c.close()


def test_two_contexts_working_side_by_side():
    """A context per direction, each on a stream of its own, queued without
    waits (what the benchmark's step does): one gathers a ResNet-sized batch
    round after round while the other scatters the responses of a LeNet-sized
    one; arenas the batches do not divide, so every call starts somewhere else.
    Arena, TX ring and both cursors are held against the oracle at the end."""
    wg, ws = synth.make_workload(2, 6), synth.make_workload(1, 300)
    dg, ds = DeviceWorkload(wg), DeviceWorkload(ws)
    cap_g = 2 * int(wg.req_sizes.sum()) + 1001
    arena_g = torch.zeros(cap_g, dtype=torch.uint8, device=DEV)
    cap_s = int(ws.resp_sizes.sum()) + 333
    resp_np = np.random.default_rng(9).integers(0, 256, cap_s, dtype=np.uint8)
    arena_s = to_dev(resp_np, DEV)
    g, s = SgContext(0, max_reqs=4096, max_frames=1 << 16), SgContext(0, max_reqs=4096, max_frames=1 << 16)
    ga = g.gather_args(dg.rx, dg.frag_slot, None, dg.req_first, dg.n_req, dg.n_frags, AppRef(arena=arena_g, cap=cap_g),
                       None, flags=capi.F_ASYNC | capi.F_RULE_FRAGS, fixed_req_size=int(wg.req_sizes[0]), mtu=wg.mtu)
    sa = s.scatter_args(ds.rx, ds.tx, ds.tx_slot, ds.hdr_src_slot, ds.resp_first, None, int(ws.resp_sizes[0]), ds.n_req,
                        ds.n_frames, ws.mtu, AppRef(arena=arena_s, cap=cap_s), None, ws.flags | capi.F_ASYNC)
    g.set_cursor(0, 77)
    s.set_cursor(1, 5)
    torch.cuda.synchronize()
    rounds = 7
    for _ in range(rounds):
        g.gather_batch_raw(ga)
        s.scatter_batch_raw(sa)
    g.sync()
    s.sync()
    want = np.zeros(cap_g, np.uint8)
    cur_g, cur_s = 77, 5
    tx = None
    for _ in range(rounds):
        want, _, cur_g = oracle.gather(wg, arena_cap=cap_g, cursor=cur_g, out=want)
        tx = ws.tx_ring_init.copy()
        _, cur_s = oracle.scatter(ws, ws.ring, tx, resp_np, arena_cap=cap_s, cursor=cur_s)
    got = arena_g.cpu().numpy()
    assert np.array_equal(got, want), first_diff(got, want)
    got = ds.tx_ring.cpu().numpy()
    assert np.array_equal(got, tx), first_diff(got, tx)
    assert g.get_cursor(0) == cur_g and s.get_cursor(1) == cur_s
    g.close()
    s.close()
