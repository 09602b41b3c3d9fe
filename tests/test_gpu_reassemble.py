"""Request reassembly on the device (sg_hip_reassemble) against the oracle's
replay of the reference's get_rr / rr_emplace_mbuf / is_rr_ready logic, and
the tables it emits feeding the gather."""
import numpy as np
import pytest
import torch

import oracle
from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, RingRef, SgContext, to_dev

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def device_reassemble(ctx, w, arrivals, len_nic=None, req_size=0, ring=None, max_reqs=8192, reset=True, flags=0):
    n = len(arrivals)
    if reset:
        ctx.reassemble_reset()  # the context is shared: nothing of an earlier case may still be in flight
    rx = RingRef(torch.from_numpy(w.ring if ring is None else ring).to(DEV), w.n_slots, w.slot_size, w.profile)
    # room for the fragments that earlier calls left in flight as well
    fs = torch.zeros(n + 4096, dtype=torch.int32, device=DEV)
    fl = torch.zeros(n + 4096, dtype=torch.int32, device=DEV)
    rf = torch.zeros(max_reqs + 1, dtype=torch.int32, device=DEV)
    tok = torch.zeros(max_reqs, dtype=torch.int64, device=DEV)
    ln = to_dev(len_nic, DEV) if len_nic is not None else None
    n_req, n_frag, n_left = ctx.reassemble(rx, to_dev(np.ascontiguousarray(arrivals, np.uint32), DEV), n, fs, fl, rf,
                                           tok, ln, req_size, flags=flags)
    return (fs[:n_frag].cpu().numpy().view(np.uint32), fl[:n_frag].cpu().numpy().view(np.uint32),
            rf[:n_req + 1].cpu().numpy().view(np.uint32), tok[:n_req].cpu().numpy().view(np.uint64), n_left, rx,
            (fs, fl, rf))


# workgroups of 1024 threads, and of 256 as for a call that runs beside a long kernel (SG_F_SMALL_GROUPS)
GROUPS = pytest.mark.parametrize("flags", [0, capi.F_SMALL_GROUPS], ids=["groups-of-1024", "groups-of-256"])


@GROUPS
@pytest.mark.parametrize("cfg,n", [(1, None), (2, 3), (2, None), (3, None), (4, 300), (4, None), (5, 2)])
def test_reassembly_matches_oracle(ctx, cfg, n, flags):
    w = synth.make_workload(cfg, n)
    print(f"case reassemble cfg={cfg} n_req={w.n_req} arrivals={len(w.arrivals)} flags={flags:#x}", flush=True)
    rng = np.random.default_rng(cfg)
    for arr in (w.arrivals, rng.permutation(w.arrivals)):
        got = device_reassemble(ctx, w, arr, flags=flags)
        want = oracle.reassemble(w, arrivals=arr)
        for g, e, name in zip(got[:4], want, ("frag_slot", "frag_len", "req_first", "req_token")):
            assert np.array_equal(g, e), name
        assert got[4] == 0


@GROUPS
def test_reassembly_ref64_by_request_size(ctx, flags):
    w = synth.make_workload(2, 4, profile=synth.HDR_REF64)
    len_nic = np.zeros(w.n_slots, np.uint32)
    len_nic[w.frag_slot] = w.frag_len
    size = int(w.req_sizes[0])
    got = device_reassemble(ctx, w, w.arrivals, len_nic=len_nic, req_size=size, flags=flags)
    want = oracle.reassemble(w, req_size=size, frag_len_nic=len_nic)
    for g, e in zip(got[:4], want):
        assert np.array_equal(g, e)


def test_lost_fragments_and_token_zero(ctx):
    """A lost fragment parks its request until the fragment comes; token 0 is
    dropped; the rest goes through."""
    w = synth.make_workload(1, 10)
    ring = w.ring.copy().reshape(w.n_slots, w.slot_size)
    zero_slot = int(w.frag_slot[int(w.req_first[3])])       # a fragment of request 3 loses its token
    ring[zero_slot, 42:50] = 0
    arr = np.delete(w.arrivals, np.flatnonzero(w.arrivals == w.frag_slot[int(w.req_first[6]) + 1]))  # request 6 loses one
    w2 = synth.make_workload(1, 10)
    w2.ring = ring.reshape(-1)
    got = device_reassemble(ctx, w2, arr, ring=w2.ring)
    want = oracle.reassemble(w2, arrivals=arr)
    for g, e in zip(got[:4], want):
        assert np.array_equal(g, e)
    assert len(got[3]) == 8
    assert got[4] == 2            # requests 3 and 6 stay in flight, each one fragment short
    assert ctx.last_dropped == 1  # the token-0 packet
    # the missing fragment of request 6 comes with the next burst: the request completes there
    late = np.array([w.frag_slot[int(w.req_first[6]) + 1]], np.uint32)
    got = device_reassemble(ctx, w2, late, ring=w2.ring, reset=False)
    assert len(got[3]) == 1 and got[3][0] == w.req_ids[6] and got[4] == 1
    assert np.array_equal(got[0], w.frag_slot[int(w.req_first[6]):int(w.req_first[7])])
    # a clean burst after a reset
    got = device_reassemble(ctx, w, w.arrivals)
    want = oracle.reassemble(w)
    for g, e in zip(got[:4], want):
        assert np.array_equal(g, e)


def test_reassemble_then_gather(ctx):
    """Arrival list in, tensor out: no per-packet work on the host."""
    w = synth.make_workload(4, 500)
    fs, fl, rf, tok, left, rx, dev_tabs = device_reassemble(ctx, w, w.arrivals)
    n_req, n_frag = len(tok), len(fs)
    cap = int(w.req_sizes.sum())
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    offs = torch.zeros(n_req + 1, dtype=torch.int64, device=DEV)
    ctx.set_cursor(0, 0)
    ctx.gather_batch(rx, dev_tabs[0], None, dev_tabs[2], n_req, n_frag, AppRef(arena=arena, cap=cap), offs)
    exp, eoffs, _ = oracle.gather(w, arena_cap=cap)
    assert np.array_equal(arena.cpu().numpy(), exp)
    assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)


def test_bad_arrival_is_refused(ctx):
    w = synth.make_workload(1, 4)
    arr = w.arrivals.copy()
    arr[2] = w.n_slots + 7
    from splitrpc_amd.engine import SgError
    with pytest.raises(SgError) as e:
        device_reassemble(ctx, w, arr)
    assert e.value.code == capi.SG_E_DATA
    got = device_reassemble(ctx, w, w.arrivals)  # and the context recovers
    assert np.array_equal(got[0], w.frag_slot)


@pytest.mark.parametrize("kind", ["echo", "vec_add"])
def test_client_requests_served_on_the_device_end_to_end(ctx, kind):
    """A burst of the reference clients' requests (REF64 headers) goes through
    reassembly, gather, the "model" and scatter on the device, and the
    clients' own checks (lib_loadgen/*_client.cc) accept every response."""
    import torch
    from splitrpc_amd import capi, loadgen
    from splitrpc_amd.engine import AppRef, DeviceWorkload, to_dev
    size, rsize = (30000, 30000) if kind == "echo" else (9000, 5000)
    w = loadgen.client_workload(kind, 37, size, resp_size=rsize, flags=synth.F_UDP_CSUM_PSEUDO | synth.F_REF_QUIRKS)
    print(f"case client {kind} n_req={w.n_req} frags={w.n_frags}", flush=True)
    dw = DeviceWorkload(w)
    dev = "cuda"
    ln = np.zeros(w.n_slots, np.uint32)
    ln[w.frag_slot] = w.frag_len
    fs = torch.zeros(w.n_frags, dtype=torch.int32, device=dev)
    fl = torch.zeros(w.n_frags, dtype=torch.int32, device=dev)
    rf = torch.zeros(8193, dtype=torch.int32, device=dev)
    ctx.reassemble_reset()
    n_req, n_frag, n_left = ctx.reassemble(dw.rx, dw.arrivals, w.n_frags, fs, fl, rf, len_nic=to_dev(ln, dev),
                                           req_size=size)
    assert (n_req, n_frag, n_left) == (w.n_req, w.n_frags, 0)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    ctx.gather_batch(dw.rx, fs, fl, rf, n_req, n_frag, dw.req_app, dw.req_offsets,
                     flags=capi.F_RULE_FRAGS, fixed_req_size=size, mtu=w.mtu)
    if kind == "echo":
        resp_app = dw.req_app
        tx, tx_slot, hsrc, first = dw.rx, fs, fs, rf          # answered in place, frame for frame
        n_frames = n_frag
    else:
        served = (dw.req_arena.view(w.n_req, size)[:, :rsize] + 1).contiguous().view(-1)   # the model
        resp_app = AppRef(arena=served, cap=int(served.numel()))
        tx, tx_slot, hsrc, first, n_frames = dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, dw.n_frames
    ctx.scatter_batch(dw.rx, tx, tx_slot, hsrc, first, None, rsize, n_req, n_frames, w.mtu, resp_app, None, w.flags)
    out = (dw.ring if kind == "echo" else dw.tx_ring).cpu().numpy()
    assert loadgen.verify_responses(w, out, kind) == 0
