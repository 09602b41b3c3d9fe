"""sg_hip_shunt_batch -- one pass of the shunter's loop, gather and scatter in
ONE launch where the two calls can share one -- against the CPU oracle's
gather followed by its scatter, bit for bit, through the C ABI: arenas, TX
ring, offsets and both bump-ring cursors, over calls in a row and over graph
replays.  Pairs of calls that cannot share a launch (long frames, short-frame
kernels, tensors against an arena, an echo answered in place) must come out the
same through the two-call path the entry point then takes."""
import numpy as np
import pytest
import torch

from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, SgContext

from helpers import expected_gather, expected_scatter, first_diff

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _args(ctx, dw, w, req_arena, req_cap, req_offs, resp_offs, flags=0, rule=True):
    """Argument blocks of a gather into `req_arena` and the workload's scatter."""
    fx = int(w.req_sizes[0])
    ga = ctx.gather_args(dw.rx, dw.frag_slot, dw.frag_len if w.profile else None, dw.req_first, dw.n_req, dw.n_frags,
                         AppRef(arena=req_arena, cap=req_cap) if req_arena is not None else dw.req_app, req_offs,
                         flags=flags | (capi.F_RULE_FRAGS if rule else 0), fixed_req_size=fx if rule else 0, mtu=w.mtu)
    rs = w.resp_sizes
    one = bool((rs == rs[0]).all())
    sa = ctx.scatter_args(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, None if one else dw.resp_size,
                          int(rs[0]) if one else 0, dw.n_req, dw.n_frames, w.mtu, dw.resp_app, resp_offs,
                          w.flags | flags)
    return ga, sa


SHARED = {
    "resnet50-2": lambda p: synth.make_workload(2, 2, profile=p),
    "three-frames": lambda p: synth.make_custom([4200] * 40, [3000] * 40, seed=71, profile=p,
                                                flags=synth.F_UDP_CSUM_PSEUDO | synth.F_IPV4_CSUM),
    "full-udp-checksum": lambda p: synth.make_custom([2800] * 33, [2799] * 33, seed=72, profile=p,
                                                     flags=synth.F_UDP_CSUM_FULL | synth.F_IPV4_CSUM),
    "one-request": lambda p: synth.make_custom([1400 * 9 + 1], [1400], seed=73, profile=p),
    # short last fragments riding in the gather's half, eight short frames to a wavefront in the scatter's
    "lenet-9": lambda p: synth.make_workload(1, 9, profile=p),
    "lenet-1500": lambda p: synth.make_workload(1, 1500, profile=p),   # 6128 wavefronts: the most that shares
}


@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64], ids=["bl58", "ref64"])
@pytest.mark.parametrize("name", list(SHARED))
def test_one_launch_moves_what_two_calls_move(name, profile):
    w = SHARED[name](profile)
    print(f"case shunt shared {name} profile={profile} n_req={w.n_req} frags={w.n_frags} frames={w.n_resp_frames}",
          flush=True)
    ctx = SgContext(0, max_reqs=8192, max_frames=1 << 17)
    dw = DeviceWorkload(w)
    total = int(w.req_sizes.sum())
    cap = 2 * total + 4096 + 10  # no whole number of batches fills the arena: the third call wraps
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    ga, sa = _args(ctx, dw, w, arena, cap, offs, dw.resp_offsets)
    rcur, tcur = 77 * 16 + 6, 0
    ctx.set_cursor(0, rcur)
    ctx.set_cursor(1, tcur)
    ctx.set_profiling(True)
    for call in range(3):
        arena.zero_()
        dw.tx_ring.copy_(torch.from_numpy(w.tx_ring_init).to(DEV))
        torch.cuda.synchronize()
        ctx.shunt_batch_raw(ga, sa)
        exp, eoffs, ecur = expected_gather(w, arena_cap=cap, cursor=rcur)
        got = arena.cpu().numpy()
        assert np.array_equal(got, exp), f"call {call}: " + first_diff(got, exp)
        assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
        assert ctx.get_cursor(0) == ecur
        exp_tx, toffs, tnext = expected_scatter(w, None, resp_cap=dw.resp_app.cap, cursor=tcur)
        got = dw.tx_ring.cpu().numpy()
        assert np.array_equal(got, exp_tx), f"call {call}: " + first_diff(got, exp_tx)
        assert np.array_equal(dw.resp_offsets.cpu().numpy().view(np.uint64), toffs)
        assert ctx.get_cursor(1) == tnext
        rcur, tcur = ecur, tnext
    # one launch per call carried both directions
    assert ctx.kernel_time(1)[1] == 3 and ctx.kernel_time(2)[1] == 0 and ctx.kernel_time(0)[1] == 0
    ctx.close()


APART = {
    # (workload, why the two calls keep kernels of their own)
    "jumbo": lambda: synth.make_workload(5, 1),                     # frames of several wavefronts
    "short-frames-16-lanes": lambda: synth.make_custom([300] * 50, [300] * 50, seed=78),  # short frames, 16 lanes each
    "bert": lambda: synth.make_workload(3, 20),                     # tensors; short last fragments
    "mixed-echo": lambda: synth.make_workload(4, 50),               # variable sizes, answered in place
    "sizes-differ": lambda: synth.make_custom([4200] * 12, [100 + 333 * k for k in range(12)], seed=74),
    # more wavefronts than the chip holds at once: faster as two calls
    "lenet-4096": lambda: synth.make_workload(1, 4096),
    "two-frames-3000": lambda: synth.make_custom([4200] * 3000, [2800] * 3000, seed=77, flags=synth.F_UDP_CSUM_PSEUDO),
}


@pytest.mark.parametrize("name", list(APART))
def test_pairs_that_cannot_share_a_launch_take_two(name):
    w = APART[name]()
    print(f"case shunt apart {name} n_req={w.n_req} frags={w.n_frags} frames={w.n_resp_frames}", flush=True)
    ctx = SgContext(0, max_reqs=8192, max_frames=1 << 17)
    dw = DeviceWorkload(w)
    one_size = bool((w.req_sizes == w.req_sizes[0]).all())
    ga, sa = _args(ctx, dw, w, None, 0, dw.req_offsets, dw.resp_offsets, rule=one_size)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    ctx.shunt_batch_raw(ga, sa)
    if w.in_tensor_sizes:
        exp, _, _ = expected_gather(w)
        for t, e in zip(dw.in_tensors, exp):
            assert np.array_equal(t.cpu().numpy(), e)
        gathered = None
    else:
        exp, eoffs, ecur = expected_gather(w, arena_cap=dw.req_app.cap)
        got = dw.req_arena.cpu().numpy()
        assert np.array_equal(got, exp), first_diff(got, exp)
        assert np.array_equal(dw.req_offsets.cpu().numpy().view(np.uint64), eoffs)
        assert ctx.get_cursor(0) == ecur
        gathered = exp
    exp_tx, toffs, tcur = expected_scatter(w, gathered, resp_cap=dw.resp_app.cap if not w.out_tensor_sizes else None)
    got = dw.tx_ring.cpu().numpy()
    assert np.array_equal(got, exp_tx), first_diff(got, exp_tx)
    if dw.resp_offsets is not None:
        assert np.array_equal(dw.resp_offsets.cpu().numpy().view(np.uint64), toffs)
        assert ctx.get_cursor(1) == tcur
    ctx.close()


def test_refusals_come_through_either_half():
    w = synth.make_custom([4200] * 6, [3000] * 6, seed=75)
    ctx = SgContext(0)
    dw = DeviceWorkload(w)
    ga, sa = _args(ctx, dw, w, None, 0, dw.req_offsets, dw.resp_offsets)
    # refused by the host before anything is launched: cursors stay
    ctx.set_cursor(0, 64)
    ctx.set_cursor(1, 0)
    keep = sa.mtu
    sa.mtu = 0
    with pytest.raises(Exception) as e:
        ctx.shunt_batch_raw(ga, sa)
    assert e.value.code == capi.SG_E_INVAL
    sa.mtu = keep
    assert ctx.get_cursor(0) == 64 and ctx.get_cursor(1) == 0
    assert ctx.lib.sg_hip_shunt_batch(ctx.h, None, None) == capi.SG_E_INVAL
    # refused by the device: a bad slot index on the gather's side is reported, the scatter's frames are out
    from splitrpc_amd.engine import to_dev
    bad = w.frag_slot.copy()
    bad[4] = w.n_slots + 3
    bad_dev = to_dev(bad, DEV)
    ga.frag_slot = bad_dev.data_ptr()
    with pytest.raises(Exception) as e:
        ctx.shunt_batch_raw(ga, sa)
    assert e.value.code == capi.SG_E_DATA
    exp_tx, _, _ = expected_scatter(w, None, resp_cap=dw.resp_app.cap)
    assert np.array_equal(dw.tx_ring.cpu().numpy(), exp_tx)
    ctx.close()


def test_shunt_calls_recorded_into_a_graph_continue_both_rings():
    """Three calls of one launch each in one graph; every replay continues both
    bump rings where the last one stopped, with eager work in between."""
    w = synth.make_custom([4200] * 10, [3000] * 10, seed=76, flags=synth.F_UDP_CSUM_PSEUDO)
    s = torch.cuda.Stream()
    ctx = SgContext(0, stream=s.cuda_stream)
    dw = DeviceWorkload(w)
    total = int(w.req_sizes.sum())
    cap = 3 * total + 1234
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    ga, sa = _args(ctx, dw, w, arena, cap, offs, dw.resp_offsets, flags=capi.F_ASYNC)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    ctx.shunt_batch_raw(ga, sa)  # warm
    ctx.sync()
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        for _ in range(3):
            ctx.shunt_batch_raw(ga, sa)
    rcur = 0
    for rep in range(4):
        arena.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for _ in range(3):
            _, eoffs, rcur = expected_gather(w, arena_cap=cap, cursor=rcur)
        got = arena.cpu().numpy()
        # the three calls of a replay lay the batch down three times, one behind the other
        c = (rcur - 3 * total) % cap
        idx = np.zeros(cap, bool)
        idx[(c + np.arange(3 * total)) % cap] = True
        lin = np.concatenate([w.req_payload] * 3)
        assert np.array_equal(got[(c + np.arange(3 * total)) % cap], lin), f"replay {rep}"
        assert not got[~idx].any()
        assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
        ctx.sync()
        assert ctx.get_cursor(0) == rcur
        assert ctx.get_cursor(1) == 0  # three whole passes over the responses
        exp_tx, _, _ = expected_scatter(w, None, resp_cap=dw.resp_app.cap)
        assert np.array_equal(dw.tx_ring.cpu().numpy(), exp_tx)
        junk = torch.full((1 << 18,), rep, dtype=torch.uint8, device=DEV)
        assert int(junk[7]) == rep
    ctx.close()
