"""Asynchronous calls recorded into a HIP graph and replayed."""
import numpy as np
import pytest
import torch

from splitrpc_amd import capi, synth
from splitrpc_amd.engine import DeviceWorkload, SgContext

from helpers import expected_gather, expected_scatter, first_diff

pytestmark = pytest.mark.gpu


def test_gather_scatter_recorded_into_a_graph_and_replayed():
    """Two steps of the
    single-batch gather + scatter are recorded on the context's stream and
    replayed; every replay is held against the oracle, with eager work and
    synchronisation between the replays."""
    w = synth.make_workload(2, 4)
    s = torch.cuda.Stream()
    ctx = SgContext(0, max_reqs=64, max_frames=8192, stream=s.cuda_stream)
    dw = DeviceWorkload(w)
    # eager result first
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    dw.gather(ctx, rule=True)
    dw.scatter(ctx)
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap)
    assert np.array_equal(dw.req_arena.cpu().numpy(), exp)
    assert np.array_equal(dw.tx_ring.cpu().numpy(), exp_tx)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        for _ in range(2):
            dw.gather(ctx, flags=capi.F_ASYNC, rule=True)
            dw.scatter(ctx, flags=capi.F_ASYNC)
    for rep in range(4):
        dw.req_arena.zero_()
        dw.tx_ring.copy_(torch.from_numpy(w.tx_ring_init).cuda())
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = dw.req_arena.cpu().numpy()
        assert np.array_equal(got, exp), f"replay {rep}: " + first_diff(got, exp)
        got = dw.tx_ring.cpu().numpy()
        assert np.array_equal(got, exp_tx), f"replay {rep}: " + first_diff(got, exp_tx)
        # eager work of the library between replays
        junk = torch.full((1 << 20,), rep, dtype=torch.uint8, device="cuda")
        assert int(junk[5]) == rep
    ctx.sync()
    ctx.close()


@pytest.mark.parametrize("mode", ["rule", "fixed", "scan"])
@pytest.mark.parametrize("calls", [1, 2, 3])
def test_replays_continue_the_bump_ring(mode, calls):
    """An arena that no whole number of batches fills and a graph of one, two
    or three gather calls: every replay takes up the cursor where the previous
    one left it, whatever the number of calls recorded (the cursor is one
    device word that only the device advances)."""
    import oracle
    from splitrpc_amd.engine import AppRef
    w = synth.make_workload(1, 8)
    batch = int(w.req_sizes.sum())
    cap = 3 * batch + 1000
    s = torch.cuda.Stream()
    ctx = SgContext(0, max_reqs=64, max_frames=8192, stream=s.cuda_stream)
    dw = DeviceWorkload(w)
    arena = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    app = AppRef(arena=arena, cap=cap)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device="cuda")
    a = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs,
                        flags=capi.F_ASYNC | (capi.F_RULE_FRAGS if mode == "rule" else 0),
                        fixed_req_size=int(w.req_sizes[0]) if mode != "scan" else 0, mtu=w.mtu)
    ctx.set_cursor(0, 0)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        for _ in range(calls):
            ctx.gather_batch_raw(a)
    want = np.zeros(cap, np.uint8)
    cur = 0
    for rep in range(5):
        g.replay()
        torch.cuda.synchronize()
        for _ in range(calls):
            want, eoffs, cur = oracle.gather(w, arena_cap=cap, cursor=cur, out=want)
        got = arena.cpu().numpy()
        assert np.array_equal(got, want), f"replay {rep}: " + first_diff(got, want)
        assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
        assert ctx.get_cursor(0) == cur
    ctx.close()
