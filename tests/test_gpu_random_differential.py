"""Randomized differential test: seeded random workloads -- sizes, MTUs, slot
sizes, header profiles, checksum flags, arrival orders, tensor-major splits,
ring alignment, cursor positions -- through every mode of the HIP path and
through the CPU oracle; everything the calls write must agree bit for bit."""
import numpy as np
import pytest
import torch

import oracle
from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, RingRef, to_dev

from helpers import first_diff

pytestmark = pytest.mark.gpu

DEV = "cuda"
ORDERS = ["in_order", "perm_within_request", "interleave_keep_order", "shuffle_all"]


def random_case(seed: int, many: bool = False):
    """``many``: hundreds to thousands of requests of a few frames each -- launches large enough for
    the XCD-aware order, the tiled scan of request totals and the several-requests-per-wavefront
    descriptor kernels -- instead of a dozen requests of any size."""
    rng = np.random.default_rng((50000 if many else 1000) + seed)
    profile = int(rng.integers(0, 2))
    hl = synth.hdr_len(profile)
    mtu = int(rng.choice([64, 256, 1400, 2000] if many else [64, 256, 1400, 1408, 2000, 4242, 8800]))
    slot_size = 2 * ((hl + mtu + int(rng.integers(0, 100 if many else 300)) + 1) // 2)
    n_req = int(rng.integers(500, 6000)) if many else int(rng.integers(1, 14))
    uniform = bool(rng.integers(0, 2))
    in_place = bool(rng.integers(0, 4) == 0)
    if uniform:
        size = int(rng.integers(1, (4 if many else 6) * mtu + 2))
        sizes = [size] * n_req
        rs = size if in_place else int(rng.integers(1, (3 if many else 5) * mtu + 2))
        resp = [rs] * n_req
    else:
        top = [mtu // 4 + 2, 2 * mtu + 2, 6 * mtu + 2][int(rng.integers(0, 3))] if many else 5 * mtu + 2
        sizes = [int(x) for x in rng.integers(0, top, n_req)]
        if rng.integers(0, 3) == 0:
            sizes[int(rng.integers(0, n_req))] = 0
        resp = list(sizes) if in_place else [int(x) for x in rng.integers(0, top if many else 4 * mtu + 2, n_req)]
        # a request without fragments has no header a response could be built from
        resp = [0 if s == 0 else r for s, r in zip(sizes, resp)]
    in_t, out_t = (), ()
    if uniform and not in_place and rng.integers(0, 3) == 0 and sizes[0] >= 4:
        cuts = sorted(set(int(x) for x in rng.integers(1, sizes[0], int(rng.integers(1, 4)))))
        bounds = [0] + cuts + [sizes[0]]
        in_t = tuple(b - a for a, b in zip(bounds[:-1], bounds[1:]))
        if rng.integers(0, 2) and resp[0] >= 2:
            c = int(rng.integers(1, resp[0]))
            out_t = (c, resp[0] - c)
    flags = int(rng.integers(0, 16))
    if (flags & synth.F_REF_QUIRKS) and not (flags & synth.F_UDP_CSUM_PSEUDO):
        flags &= ~synth.F_REF_QUIRKS
    frames = sum(synth.num_frames(s, mtu) for s in sizes)
    n_slots = max(frames, 1) + int(rng.integers(0, 5))
    w = synth.make_custom(sizes, resp, mtu=mtu, slot_size=slot_size, n_slots=n_slots,
                          order=str(rng.choice(ORDERS)), seed=seed, profile=profile, in_tensor_sizes=in_t,
                          out_tensor_sizes=out_t, flags=flags, in_place=in_place,
                          head=int(rng.integers(0, n_slots)))
    shift = int(rng.choice([0, 0, 2, 4, 8, 10]))
    return w, uniform, shift, rng


@pytest.mark.parametrize("seed,many", [(s, False) for s in range(300)] + [(s, True) for s in range(16)],
                         ids=[str(s) for s in range(300)] + [f"many-{s}" for s in range(16)])
def test_random_workload(ctx, seed, many):
    w, uniform, shift, rng = random_case(seed, many)
    ref64 = w.profile == synth.HDR_REF64
    print(f"case random seed={seed} many={many} n_req={w.n_req} frags={w.n_frags} frames={w.n_resp_frames} mtu={w.mtu} "
          f"slot={w.slot_size} profile={w.profile} flags={w.flags} in_place={w.tx_in_place} "
          f"tensors={w.in_tensor_sizes}/{w.out_tensor_sizes} shift={shift}", flush=True)
    dw = DeviceWorkload(w, ring_shift=shift)
    # ---- reassembly of the burst: the tables must come out as the generator staged them
    # (completion order; requests without fragments never arrive)
    if w.n_frags and (not ref64 or uniform):
        fs = torch.zeros(w.n_frags, dtype=torch.int32, device=DEV)
        fl = torch.zeros(w.n_frags, dtype=torch.int32, device=DEV)
        rf = torch.zeros(8193, dtype=torch.int32, device=DEV)
        tok = torch.zeros(8192, dtype=torch.int64, device=DEV)
        ln = np.zeros(w.n_slots, np.uint32)
        ln[w.frag_slot] = w.frag_len
        got = ctx.reassemble(dw.rx, dw.arrivals, w.n_frags, fs, fl, rf, req_token=tok,
                             len_nic=to_dev(ln, DEV) if (ref64 or seed % 2) else None,
                             req_size=int(w.req_sizes[0]) if ref64 else 0)
        per = (w.req_first[1:] - w.req_first[:-1]).astype(np.int64)
        live = per > 0
        assert got == (int(live.sum()), w.n_frags, 0)
        # the oracle's replay of the receive path on the same arrivals
        efs, efl, erf, etok = oracle.reassemble(w, req_size=int(w.req_sizes[0]) if ref64 else 0,
                                                frag_len_nic=ln if (ref64 or seed % 2) else None)
        assert np.array_equal(fs.cpu().numpy().view(np.uint32), efs)
        assert np.array_equal(fl.cpu().numpy().view(np.uint32), efl)
        assert np.array_equal(rf.cpu().numpy().view(np.uint32)[:len(erf)], erf)
        assert np.array_equal(tok.cpu().numpy().view(np.uint64)[:len(etok)], etok)
        assert np.array_equal(fs.cpu().numpy().view(np.uint32), w.frag_slot.astype(np.uint32))
        assert np.array_equal(fl.cpu().numpy().view(np.uint32), w.frag_len.astype(np.uint32))
        want_first = np.concatenate([[0], np.cumsum(per[live])]).astype(np.uint32)
        assert np.array_equal(rf.cpu().numpy().view(np.uint32)[:len(want_first)], want_first)
        assert np.array_equal(tok.cpu().numpy().view(np.uint64)[:int(live.sum())], w.req_ids[live])

    modes = [(False, False)] + ([(True, False), (True, True)] if uniform else [])
    packed_req = not w.in_tensor_sizes
    for fixed, rule in modes:
        # ---- gather
        cur0 = 0
        if packed_req:
            cap = dw.req_app.cap + int(rng.integers(0, 3)) * 777
            cur0 = int(rng.integers(0, cap))
            arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
            app = AppRef(arena=arena, cap=cap)
            offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
            ctx.set_cursor(0, cur0)
        else:
            for t in dw.in_tensors:
                t.zero_()
            app, offs = dw.req_app, None
        size0 = int(w.req_sizes[0]) if (fixed and w.n_req) else 0
        ctx.gather_batch(dw.rx, dw.frag_slot, dw.frag_len if (ref64 or seed % 3 == 0) else None, dw.req_first,
                         dw.n_req, dw.n_frags, app, offs, flags=capi.F_RULE_FRAGS if rule else 0,
                         fixed_req_size=size0, mtu=w.mtu if rule else 0)
        if packed_req:
            exp, eoffs, ecur = oracle.gather(w, arena_cap=cap, cursor=cur0, use_frag_len=True)
            got = arena.cpu().numpy()
            assert np.array_equal(got, exp), f"gather fixed={fixed} rule={rule}: " + first_diff(got, exp)
            assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
            assert ctx.get_cursor(0) == ecur
        else:
            exp, _, _ = oracle.gather(w, use_frag_len=True)
            for t, e in zip(dw.in_tensors, exp):
                assert np.array_equal(t.cpu().numpy(), e)

        # ---- scatter
        if w.n_resp_frames == 0:
            continue
        fuse = rule
        if w.tx_in_place:
            # echo out of the arena the gather just filled, from the same cursor
            rapp, rcur, src, rcap = app, cur0, exp, cap
            tx_exp = w.ring.copy()
            rx_exp = tx_exp
            dw.ring.copy_(to_dev(w.ring, DEV))
        elif w.out_tensor_sizes:
            rapp, rcur, rcap = dw.resp_app, 0, None
            per = int(sum(w.out_tensor_sizes))
            rp = w.resp_payload.reshape(w.n_req, per)
            src, o = [], 0
            for s in w.out_tensor_sizes:
                src.append(np.ascontiguousarray(rp[:, o:o + s]).reshape(-1))
                o += s
            tx_exp, rx_exp = w.tx_ring_init.copy(), w.ring
            dw.tx_ring.copy_(to_dev(w.tx_ring_init, DEV))
        else:
            rcap = dw.resp_app.cap
            rcur = int(rng.integers(0, rcap))
            rolled = np.roll(np.resize(w.resp_payload, rcap) if w.resp_payload.size < rcap else w.resp_payload, rcur)
            rarena = to_dev(rolled, DEV)
            rapp, src = AppRef(arena=rarena, cap=rcap), rolled
            tx_exp, rx_exp = w.tx_ring_init.copy(), w.ring
            dw.tx_ring.copy_(to_dev(w.tx_ring_init, DEV))
        ctx.set_cursor(1, rcur)
        rs0 = int(w.resp_sizes[0]) if fixed else 0
        ctx.scatter_batch(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first,
                          None if fixed else dw.resp_size, rs0, dw.n_req, dw.n_frames, w.mtu, rapp, None,
                          w.flags | (0 if fuse else capi.F_NO_FUSE))
        oracle.scatter(w, rx_exp, tx_exp, src, arena_cap=rcap, cursor=rcur, fixed_size=rs0 if fixed else None)
        got = dw.tx_ring.cpu().numpy()
        assert np.array_equal(got, tx_exp), f"scatter fixed={fixed} fuse={fuse}: " + first_diff(got, tx_exp)
        if w.tx_in_place:
            dw.ring.copy_(to_dev(w.ring, DEV))  # the echo overwrote the request headers: restore for the next mode
