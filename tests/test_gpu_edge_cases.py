"""Edge cases of the HIP path through the C ABI: every alignment phase, the
per-request entry points, the reference's own 64-byte header profile, ragged
and empty tables, wrap-around arenas, refused input, and size-independent
properties at the benchmark's full sizes.  Bit-exact against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, RingRef, SgContext, SgError, to_dev

from helpers import conn_templates, expected_gather, expected_scatter, first_diff

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev_u8(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


# ---------------------------------------------------------------- per-request entry points

def test_copy_runs_every_phase_and_length(ctx):
    """sg_hip_gather / sg_hip_scatter: host-built run tables, all 16 x 16
    source/destination phases, lengths around every chunk boundary."""
    rng = np.random.default_rng(100)
    src_h = rng.integers(0, 256, 1 << 20, dtype=np.uint8)
    src = dev_u8(src_h)
    dst = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    want = np.zeros(1 << 20, np.uint8)
    lens = [0, 1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 112, 1007, 1008, 1009, 1400, 2016, 2017, 2032,
            4095, 8800]
    runs, so, do = [], 64, 64
    for sp in range(16):
        for dp in range(16):
            ln = lens[(sp * 16 + dp) % len(lens)]
            s = (so + 15) // 16 * 16 + sp
            d = (do + 15) // 16 * 16 + dp
            runs.append((s, d, ln))
            want[d:d + ln] = src_h[s:s + ln]
            so, do = s + ln + 40, d + ln + 40
    print(f"case copy_runs: {len(runs)} runs", flush=True)
    for scatter in (False, True):
        dst.zero_()
        for k in range(0, len(runs), 500):
            part = runs[k:k + 500]
            ctx.copy_runs([src.data_ptr() + s for s, _, _ in part], [dst.data_ptr() + d for _, d, _ in part],
                          [n for _, _, n in part], scatter=scatter)
        got = dst.cpu().numpy()
        assert np.array_equal(got, want), first_diff(got, want)


def test_copy_runs_long_run_is_cut(ctx):
    rng = np.random.default_rng(101)
    n = 3_000_003
    src_h = rng.integers(0, 256, n + 64, dtype=np.uint8)
    src, dst = dev_u8(src_h), torch.zeros(n + 64, dtype=torch.uint8, device=DEV)
    ctx.copy_runs([src.data_ptr() + 3], [dst.data_ptr() + 9], [n])
    got = dst.cpu().numpy()
    assert np.array_equal(got[9:9 + n], src_h[3:3 + n]) and not got[:9].any() and not got[9 + n:].any()


def test_run_table_overflow_is_refused(ctx):
    skb = capi.SkBuf()
    skb.num_items = 1024  # len[] holds 1023 (src/p2p_bufs.h:37)
    rc = ctx.lib.sg_hip_gather(ctx.h, C.byref(skb))
    assert rc == capi.SG_E_INVAL


@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64])
@pytest.mark.parametrize("flags", [0, synth.F_UDP_CSUM_PSEUDO, synth.F_UDP_CSUM_PSEUDO | synth.F_REF_QUIRKS,
                                   synth.F_IPV4_CSUM | synth.F_UDP_CSUM_PSEUDO])
def test_swap_hdrs_in_place(ctx, profile, flags):
    """sg_hip_swap_hdrs against swap + routing + lengths + sums of the oracle."""
    rng = np.random.default_rng(102 + flags)
    n, slot = 37, 256
    hl = synth.hdr_len(profile)
    buf = rng.integers(0, 256, n * slot, dtype=np.uint8)
    buf.reshape(n, slot)[:, 14] = 0x45
    dev = dev_u8(buf)
    payload_size, mtu = 36 * 1400 + 333, 1400
    ctx.swap_hdrs([dev.data_ptr() + i * slot for i in range(n)], profile, payload_size, mtu, flags)
    want = buf.copy().reshape(n, slot)
    L = oracle.lib()
    for i in range(n):
        h = want[i, :64].copy()
        L.sgo_rewrite_resp_hdr(h.ctypes.data_as(C.c_void_p), profile, flags, i, n,
                               L.sgo_frame_len(payload_size, mtu, i))
        want[i, :hl] = h[:hl]
    got = dev.cpu().numpy().reshape(n, slot)
    assert np.array_equal(got, want), first_diff(got.reshape(-1), want.reshape(-1))


@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64])
@pytest.mark.parametrize("flags", [0, synth.F_UDP_CSUM_PSEUDO | synth.F_REF_QUIRKS,
                                   synth.F_IPV4_CSUM | synth.F_UDP_CSUM_PSEUDO])
def test_set_hdrs_from_template(ctx, profile, flags):
    """sg_hip_set_hdrs against the oracle's rr_set_hdr."""
    rng = np.random.default_rng(300 + flags)
    n, slot = 23, 128
    hl = synth.hdr_len(profile)
    buf = rng.integers(0, 256, n * slot, dtype=np.uint8)
    tmpl = rng.integers(0, 256, 64, dtype=np.uint8)
    tmpl[14] = 0x45
    token = 0x0123456789abcdef
    dev = dev_u8(buf)
    payload_size, mtu = 22 * 1400 + 1, 1400
    ctx.set_hdrs([dev.data_ptr() + i * slot for i in range(n)], tmpl.tobytes(), token, profile,
                 payload_size, mtu, flags)
    want = buf.copy().reshape(n, slot)
    L = oracle.lib()
    for i in range(n):
        h = np.zeros(64, np.uint8)
        L.sgo_template_resp_hdr(h.ctypes.data_as(C.c_void_p), tmpl.ctypes.data_as(C.c_void_p), profile, flags,
                                token, i, n, L.sgo_frame_len(payload_size, mtu, i))
        want[i, :hl] = h[:hl]
    got = dev.cpu().numpy().reshape(n, slot)
    assert np.array_equal(got, want), first_diff(got.reshape(-1), want.reshape(-1))


# ---------------------------------------------------------------- header profiles, flags

@pytest.mark.parametrize("cfg,n", [(1, 9), (2, 2), (5, 1)])
@pytest.mark.parametrize("extra", [0, synth.F_REF_QUIRKS, synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL])
def test_ref64_profile(ctx, cfg, n, extra):
    """The reference's own p2p_rpc_hdr: 64 bytes, lengths from the NIC table."""
    w = synth.make_workload(cfg, n, profile=synth.HDR_REF64)
    w.flags |= extra
    print(f"case ref64 cfg={cfg} n={n} flags={w.flags}", flush=True)
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    dw.gather(ctx, use_frag_len=True)
    exp, offs, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    assert np.array_equal(dw.req_arena.cpu().numpy(), exp)
    dw.scatter(ctx)
    exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap)
    got = dw.tx_ring.cpu().numpy()
    assert np.array_equal(got, exp_tx), first_diff(got, exp_tx)


@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64])
@pytest.mark.parametrize("flags", [0, synth.F_UDP_CSUM_PSEUDO | synth.F_REF_QUIRKS,
                                   synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL])
@pytest.mark.parametrize("with_tokens", [True, False])
def test_headers_from_connection_templates(ctx, profile, flags, with_tokens):
    """Fresh response buffers: headers copied from per-request templates."""
    w = synth.make_custom([5000, 77, 1400, 0, 1401, 60000], [3000, 1, 1400, 0, 2801, 4200], seed=77,
                          flags=flags, profile=profile)
    print(f"case templates profile={profile} flags={flags} tokens={with_tokens}", flush=True)
    dw = DeviceWorkload(w)
    tm, tk = conn_templates(w, seed=5)
    if with_tokens:
        tk = tk ^ np.uint64(0x5a5a00000000a5a5)   # tokens that differ from the templates' own
    d_tm = to_dev(tm.reshape(-1), "cuda")
    d_tk = to_dev(tk, "cuda") if with_tokens else None
    ctx.set_cursor(0, 0)
    dw.gather(ctx, use_frag_len=profile == synth.HDR_REF64)
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    for fuse in (True, False):
        for fixed in (False,):
            ctx.set_cursor(1, 0)
            dw.tx_ring.copy_(to_dev(w.ring if w.tx_in_place else w.tx_ring_init, "cuda"))
            dw.scatter(ctx, fuse=fuse, fixed=fixed, templates=d_tm, tokens=d_tk)
            exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap, templates=tm,
                                            tokens=tk if with_tokens else None)
            got = dw.tx_ring.cpu().numpy()
            assert np.array_equal(got, exp_tx), first_diff(got, exp_tx)


def test_ref64_without_length_table_is_refused(ctx):
    w = synth.make_workload(1, 2, profile=synth.HDR_REF64)
    dw = DeviceWorkload(w)
    with pytest.raises(SgError) as e:
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app)
    assert e.value.code == capi.SG_E_INVAL


@pytest.mark.parametrize("flags", [0, 1, 2, 3, 4, 5, 6, 7, 10, 15])
def test_every_checksum_flag_combination(ctx, flags):
    w = synth.make_custom([5000, 77, 1400, 1401, 9], [3000, 1, 1400, 2801, 4200], seed=40 + flags, flags=flags)
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    dw.gather(ctx)
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    assert np.array_equal(dw.req_arena.cpu().numpy(), exp)
    dw.scatter(ctx)
    exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap)
    got = dw.tx_ring.cpu().numpy()
    assert np.array_equal(got, exp_tx), first_diff(got, exp_tx)


# ---------------------------------------------------------------- ragged, empty, large

def test_ragged_sizes_one_byte_to_many_fragments(ctx):
    # last: 1023 fragments, what a reference run table can describe (len[] has 1023 entries)
    sizes = [1, 2, 15, 16, 17, 57, 58, 59, 1399, 1400, 1401, 2799, 2800, 2801, 70000, 3, 1432200]
    resp = [s // 3 + 1 for s in sizes]
    w = synth.make_custom(sizes, resp, seed=7, flags=synth.F_UDP_CSUM_PSEUDO | synth.F_IPV4_CSUM)
    assert int((w.req_first[1:] - w.req_first[:-1]).max()) == 1023
    print(f"case ragged frags={w.n_frags}", flush=True)
    dw = DeviceWorkload(w)
    for fixed in (False, True):
        ctx.set_cursor(0, 0)
        ctx.set_cursor(1, 0)
        dw.req_arena.zero_()
        dw.gather(ctx, fixed=fixed)
        exp, offs, cur = expected_gather(w, arena_cap=dw.req_app.cap)
        got = dw.req_arena.cpu().numpy()
        assert np.array_equal(got, exp), first_diff(got, exp)
        assert np.array_equal(dw.req_offsets.cpu().numpy().view(np.uint64), offs)
        dw.scatter(ctx, fixed=fixed)
        exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap)
        assert np.array_equal(dw.tx_ring.cpu().numpy(), exp_tx)


def test_empty_requests_and_empty_batch(ctx):
    """Requests without fragments move nothing and take no arena space."""
    w = synth.make_custom([3000, 100, 4500], [10, 10, 10], seed=9)
    dw = DeviceWorkload(w)
    # CSR with empty requests interleaved: [r0, -, r1, -, -, r2, -]
    f = w.req_first.astype(np.uint32)
    first = np.array([f[0], f[1], f[1], f[2], f[2], f[2], f[3], f[3]], np.uint32)
    n_req = len(first) - 1
    offs = torch.zeros(n_req + 1, dtype=torch.int64, device=DEV)
    ctx.set_cursor(0, 0)
    ctx.gather_batch(dw.rx, dw.frag_slot, None, to_dev(first, DEV), n_req, dw.n_frags, dw.req_app, offs)
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    assert np.array_equal(dw.req_arena.cpu().numpy(), exp)
    o = offs.cpu().numpy().view(np.uint64).tolist()
    s0, s1, s2 = (int(x) for x in w.req_sizes)  # batch order is completion order
    end = (s0 + s1 + s2) % dw.req_app.cap
    assert o == [0, s0, s0, s0 + s1, s0 + s1, s0 + s1, end, end]
    # n_req == 0 is a no-op
    ctx.gather_batch(dw.rx, dw.frag_slot, None, to_dev(first, DEV), 0, 0, dw.req_app)


# ---------------------------------------------------------------- arena wrap, cursor persistence

@pytest.mark.parametrize("mode", ["scan", "rule"])
def test_arena_wrap_and_cursor_persistence(ctx, mode):
    """Two calls in a row continue the bump ring; a request that crosses the end
    of an arena mapped once is split byte-exactly."""
    rule = mode == "rule"
    sizes = [4200] * 5 if rule else [3000, 5000, 700, 4100, 2222]
    w = synth.make_custom(sizes, [64] * 5, seed=10)
    total = int(sum(sizes))
    cap = total + 1234
    dw = DeviceWorkload(w)
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    app = AppRef(arena=arena, cap=cap)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    cur = cap - 5000  # the second request of the first call crosses the end
    ctx.set_cursor(0, cur)
    want = np.zeros(cap, np.uint8)
    for call in range(3):
        flags = capi.F_RULE_FRAGS if rule else 0
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs,
                         flags=flags, fixed_req_size=sizes[0] if rule else 0, mtu=w.mtu)
        exp, eoffs, ecur = oracle.gather(w, arena_cap=cap, cursor=cur, out=want)
        got = arena.cpu().numpy()
        assert np.array_equal(got, exp), f"call {call}: " + first_diff(got, exp)
        assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
        assert ctx.get_cursor(0) == ecur
        cur = ecur


@pytest.mark.parametrize("shift", [2, 6, 14])
@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64])
def test_rings_at_even_addresses_off_word_alignment(ctx, shift, profile):
    """A ring only has to start at an even address: every header word then
    sits at an address = 2 (mod 4).  All three gather modes, scatter and
    reassembly must read the same bytes as on an aligned ring."""
    w = synth.make_custom([4200] * 7, [3000] * 7, seed=60 + shift, profile=profile,
                          flags=synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL)
    print(f"case shifted ring shift={shift} profile={profile}", flush=True)
    dw = DeviceWorkload(w, ring_shift=shift)
    assert dw.ring.data_ptr() % 4 == 2
    exp, offs, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    ref64 = profile == synth.HDR_REF64
    for mode in ("scan", "fixed", "rule"):
        ctx.set_cursor(0, 0)
        dw.req_arena.zero_()
        dw.gather(ctx, use_frag_len=ref64, fixed=mode != "scan", rule=mode == "rule")
        got = dw.req_arena.cpu().numpy()
        assert np.array_equal(got, exp), mode + ": " + first_diff(got, exp)
    for fuse in (True, False):
        ctx.set_cursor(1, 0)
        dw.scatter(ctx, fuse=fuse)
        exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap)
        got = dw.tx_ring.cpu().numpy()
        assert np.array_equal(got, exp_tx), first_diff(got, exp_tx)
    # reassembly reads tokens and sequence numbers from the same headers
    fs = torch.zeros(w.n_frags, dtype=torch.int32, device=DEV)
    fl = torch.zeros(w.n_frags, dtype=torch.int32, device=DEV)
    rf = torch.zeros(8193, dtype=torch.int32, device=DEV)
    len_nic = None
    if ref64:
        ln = np.zeros(w.n_slots, np.uint32)
        ln[w.frag_slot] = w.frag_len
        len_nic = to_dev(ln, DEV)
    n_req, n_frag, n_left = ctx.reassemble(dw.rx, dw.arrivals, int(dw.arrivals.numel()), fs, fl, rf,
                                           len_nic=len_nic, req_size=4200 if ref64 else 0)
    assert (n_req, n_frag, n_left) == (w.n_req, w.n_frags, 0)
    assert np.array_equal(fs.cpu().numpy().view(np.uint32), w.frag_slot.astype(np.uint32))
    assert np.array_equal(fl.cpu().numpy().view(np.uint32), w.frag_len.astype(np.uint32))


@pytest.mark.parametrize("mode", ["scan", "fixed", "rule"])
def test_batch_larger_than_its_arena_is_refused(ctx, mode):
    """Such a batch would lap itself: its first and last requests would share
    bytes, written in no particular order.  Nothing is moved.  With a declared
    request size the host refuses the call; with scanned sizes the device does."""
    rule = mode == "rule"
    declared = mode != "scan"
    sizes = [4200] * 5 if declared else [3000, 5000, 700, 4100, 2222]
    w = synth.make_custom(sizes, [64] * 5, seed=11)
    cap = int(sum(sizes)) - 1
    dw = DeviceWorkload(w)
    arena = torch.full((cap,), 7, dtype=torch.uint8, device=DEV)
    ctx.set_cursor(0, 0)
    with pytest.raises(SgError) as e:
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, AppRef(arena=arena, cap=cap),
                         flags=capi.F_RULE_FRAGS if rule else 0, fixed_req_size=sizes[0] if declared else 0, mtu=w.mtu)
    assert e.value.code == (capi.SG_E_INVAL if declared else capi.SG_E_DATA)
    assert bool((arena == 7).all())
    assert ctx.get_cursor(0) == 0, "a refused batch does not advance the bump ring"
    # one byte more and it fits
    ctx.set_cursor(0, 0)
    arena2 = torch.zeros(cap + 1, dtype=torch.uint8, device=DEV)
    ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, AppRef(arena=arena2, cap=cap + 1),
                     flags=capi.F_RULE_FRAGS if rule else 0, fixed_req_size=sizes[0] if declared else 0, mtu=w.mtu)
    exp, _, _ = oracle.gather(w, arena_cap=cap + 1)
    assert np.array_equal(arena2.cpu().numpy(), exp)


def test_cursor_after_a_rule_batch_with_a_bad_last_slot(ctx):
    """A rule batch whose LAST fragment names a slot beyond the ring: that
    fragment is dropped and the call reports SG_E_DATA, but the bump ring still
    advances by the whole batch (the advance does not depend on the tables), so
    the next batch lands where the host-side ring says it does."""
    sizes = [4200] * 6
    w = synth.make_custom(sizes, [64] * 6, seed=77)
    dw = DeviceWorkload(w)
    cap = 3 * int(sum(sizes)) + 100
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    app = AppRef(arena=arena, cap=cap)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    bad = w.frag_slot.copy()
    bad[-1] = w.n_slots + 1
    start = cap - 9000
    ctx.set_cursor(0, start)
    with pytest.raises(SgError) as e:
        ctx.gather_batch(dw.rx, to_dev(bad, DEV), None, dw.req_first, dw.n_req, dw.n_frags, app, offs,
                         flags=capi.F_RULE_FRAGS, fixed_req_size=sizes[0], mtu=w.mtu)
    assert e.value.code == capi.SG_E_DATA
    want = np.zeros(cap, np.uint8)
    _, eoffs, cur = oracle.gather(w, arena_cap=cap, cursor=start, out=want)
    assert ctx.get_cursor(0) == cur
    assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
    # every fragment but the dropped one is in place
    got = arena.cpu().numpy()
    last_len = int(w.frag_len[-1])
    hole = (int(eoffs[-2]) + sizes[0] - last_len + np.arange(last_len)) % cap
    keep = np.ones(cap, bool)
    keep[hole] = False
    assert np.array_equal(got[keep], want[keep])
    # and the next batch continues from there
    ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs,
                     flags=capi.F_RULE_FRAGS, fixed_req_size=sizes[0], mtu=w.mtu)
    want, eoffs, cur2 = oracle.gather(w, arena_cap=cap, cursor=cur, out=want)
    assert ctx.get_cursor(0) == cur2
    assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
    got = arena.cpu().numpy()
    assert np.array_equal(got[keep], want[keep])


def test_odd_arena_base_and_tensor_major_split(ctx):
    """Destination phases other than the allocator's: arena and tensors at odd
    byte offsets; a fragment that straddles the tensor boundary is split."""
    w = synth.make_workload(3, 33)
    dw = DeviceWorkload(w)
    for shift in (1, 7, 8, 13):
        backing = [torch.zeros(w.n_req * s + 64, dtype=torch.uint8, device=DEV) for s in w.in_tensor_sizes]
        tensors = [b[shift:shift + w.n_req * s] for b, s in zip(backing, w.in_tensor_sizes)]
        app = AppRef(tensors=tensors, sizes=w.in_tensor_sizes)
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app)
        exp, _, _ = expected_gather(w)
        for t, e, b in zip(tensors, exp, backing):
            assert np.array_equal(t.cpu().numpy(), e)
            bb = b.cpu().numpy()
            assert not bb[:shift].any() and not bb[shift + e.size:].any()  # nothing written outside


@pytest.mark.parametrize("tensor_sizes", [(1024, 1024), (1008, 1040), (1000, 1056), (16, 2032), (700, 700, 648)])
def test_fragment_between_two_tensors_with_the_rule_declared(ctx, tensor_sizes):
    """Requests of one size cut by the rule into tensor-major buffers: the
    fragment that runs from one tensor into the next moves as one run with a
    break in its destination where both shares lie on chunk boundaries, as two
    runs where they do not, byte by byte across three tensors -- at tensor
    bases of several phases, so that all of these occur."""
    size = int(sum(tensor_sizes))
    n = 37
    w = synth.make_custom([size] * n, [64] * n, order="shuffle_all", seed=11, in_tensor_sizes=tensor_sizes)
    dw = DeviceWorkload(w)
    exp, _, _ = expected_gather(w)
    for shift in (0, 8, 3):
        backing = [torch.full((n * s + 64,), 0xEE, dtype=torch.uint8, device=DEV) for s in tensor_sizes]
        tensors = [b[shift:shift + n * s] for b, s in zip(backing, tensor_sizes)]
        app = AppRef(tensors=tensors, sizes=list(tensor_sizes))
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app,
                         flags=capi.F_RULE_FRAGS, fixed_req_size=size, mtu=w.mtu)
        for t, e, b in zip(tensors, exp, backing):
            got = t.cpu().numpy()
            assert np.array_equal(got, e), f"shift {shift}: " + first_diff(got, e)
            bb = b.cpu().numpy()
            assert (bb[:shift] == 0xEE).all() and (bb[shift + e.size:] == 0xEE).all()  # nothing written outside


# ---------------------------------------------------------------- refused input

def test_bad_slot_index_refuses_the_whole_batch(ctx):
    w = synth.make_workload(1, 4)
    dw = DeviceWorkload(w)
    bad = w.frag_slot.copy()
    bad[5] = w.n_slots + 3
    dw.req_arena.fill_(0xAB)
    ctx.set_cursor(0, 0)
    with pytest.raises(SgError) as e:
        ctx.gather_batch(dw.rx, to_dev(bad, DEV), None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app,
                         dw.req_offsets)
    assert e.value.code == capi.SG_E_DATA
    assert bool((dw.req_arena == 0xAB).all()), "a refused batch must move nothing"
    # the context is usable again afterwards
    ctx.set_cursor(0, 0)
    dw.gather(ctx)
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    assert np.array_equal(dw.req_arena.cpu().numpy(), exp)


def test_bad_tables_and_sizes_are_refused(ctx):
    w = synth.make_workload(1, 4)
    dw = DeviceWorkload(w)
    first = w.req_first.copy()
    first[2] = first[3] + 1  # not monotone
    with pytest.raises(SgError) as e:
        ctx.gather_batch(dw.rx, dw.frag_slot, None, to_dev(first, DEV), dw.n_req, dw.n_frags, dw.req_app)
    assert e.value.code == capi.SG_E_DATA
    # a header that claims more payload than a slot holds
    ring = w.ring.copy().reshape(w.n_slots, w.slot_size)
    ring[int(w.frag_slot[1]), 54:58] = np.frombuffer((5000).to_bytes(4, "little"), np.uint8)
    rx = RingRef(dev_u8(ring.reshape(-1)), w.n_slots, w.slot_size, w.profile)
    with pytest.raises(SgError) as e:
        ctx.gather_batch(rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app)
    assert e.value.code == capi.SG_E_DATA
    # declared fragmenting rule that the ring does not follow
    with pytest.raises(SgError) as e:
        ctx.gather_batch(rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app,
                         flags=capi.F_RULE_FRAGS, fixed_req_size=3136, mtu=1400)
    assert e.value.code == capi.SG_E_DATA
    # sizes beyond what the context was created for
    small = SgContext(0, max_reqs=2, max_frames=4)
    with pytest.raises(SgError) as e:
        small.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app)
    assert e.value.code == capi.SG_E_INVAL
    small.close()
    # response frame count that disagrees with size / mtu
    with pytest.raises(SgError) as e:
        ctx.scatter_batch(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first,
                          to_dev(np.full(w.n_req, 5000, np.uint64), DEV), 0, dw.n_req, dw.n_frames, w.mtu,
                          dw.resp_app, flags=capi.F_NO_FUSE)
    assert e.value.code == capi.SG_E_DATA


# ---------------------------------------------------------------- properties at full size

def be_sum_rows(rows: np.ndarray) -> np.ndarray:
    a = rows.astype(np.uint64)
    if a.shape[1] & 1:
        a = np.concatenate([a, np.zeros((a.shape[0], 1), np.uint64)], axis=1)
    s = ((a[:, 0::2] << 8) | a[:, 1::2]).sum(axis=1)
    for _ in range(4):
        s = (s & 0xFFFF) + (s >> 16)
    return s


@pytest.mark.parametrize("layout", ["arena", "arena-wrap", "tensor"])
@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64])
def test_long_frames_summed_by_several_wavefronts(ctx, layout, profile):
    """Jumbo response frames with the full UDP checksum: the payload sum of a
    frame is put together from the partial sums of the wavefronts that copy its
    sub-runs.  Both scatter kernels (rule declared / descriptor path), twice in
    a row (the accumulators must be back at zero), with a response that crosses
    the end of an arena mapped once, and with tensor-major outputs."""
    flags = synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL
    if layout == "tensor":
        resp = [26400] * 5
        w = synth.make_custom([100] * 5, resp, mtu=8800, slot_size=9216, seed=91, profile=profile, flags=flags,
                              out_tensor_sizes=[10000, 16400])
    else:
        resp = [26401] * 5
        w = synth.make_custom([100] * 5, resp, mtu=8800, slot_size=9216, seed=92, profile=profile, flags=flags)
    print(f"case long summed frames layout={layout} profile={profile}", flush=True)
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    dw.gather(ctx, use_frag_len=profile == synth.HDR_REF64)
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    start = 0
    if layout == "arena-wrap":
        # rotate the response arena so that the batch starts 30000 bytes before its end
        cap = dw.resp_app.cap
        start = cap - 30000
        dw.resp_arena.copy_(torch.roll(dw.resp_arena.clone(), start))
    for fuse in (True, False, True):
        ctx.set_cursor(1, start)
        dw.tx_ring.copy_(to_dev(w.tx_ring_init, DEV))
        dw.scatter(ctx, fuse=fuse)
        if layout == "arena-wrap":
            tx = w.tx_ring_init.copy()
            src = np.roll(w.resp_payload, start)
            oracle.scatter(w, w.ring, tx, src, arena_cap=cap, cursor=start)
            exp_tx = tx
        else:
            exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap)
        got = dw.tx_ring.cpu().numpy()
        assert np.array_equal(got, exp_tx), f"fuse={fuse}: " + first_diff(got, exp_tx)


def test_full_size_jumbo_checksums_verify(ctx):
    """Workload 5 at full size: every response frame's IPv4 and UDP checksum
    verifies to 0xffff the way a receiver would check it (RFC 1071 / 768), and
    payload bytes round-trip."""
    w = synth.make_workload(5)
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    dw.gather(ctx, rule=True)
    assert np.array_equal(dw.req_arena.cpu().numpy(), w.req_payload)
    dw.scatter(ctx)
    tx = dw.tx_ring.cpu().numpy().reshape(w.tx_n_slots, w.slot_size)
    frames = tx[w.tx_slot]
    assert bool((be_sum_rows(frames[:, 14:34]) == 0xFFFF).all())
    lens = np.concatenate([synth.frame_lens(int(s), w.mtu) for s in w.resp_sizes])
    for ln in np.unique(lens):
        sel = frames[lens == ln]
        ulen = 8 + 16 + int(ln)
        psd = np.concatenate([sel[:, 26:34], np.zeros((len(sel), 1), np.uint8), sel[:, 23:24],
                              np.full((len(sel), 1), ulen >> 8, np.uint8),
                              np.full((len(sel), 1), ulen & 0xFF, np.uint8)], axis=1)
        seg = sel[:, 34:34 + ulen]
        both = np.concatenate([psd, seg], axis=1)
        assert bool((be_sum_rows(both) == 0xFFFF).all()), f"UDP checksum of {ln}-byte frames"
    # payload of the responses, frame by frame
    off = 0
    for r in range(w.n_req):
        for i, ln in enumerate(synth.frame_lens(int(w.resp_sizes[r]), w.mtu)):
            f = int(w.resp_first[r]) + i
            if i in (0, 57, 119):
                assert np.array_equal(tx[w.tx_slot[f], 58:58 + ln], w.resp_payload[off:off + ln])
            off += int(ln)


def test_full_size_mixed_echo_round_trip(ctx):
    """Workload 4 at full size: gather, echo in place, gather again -- the same
    bytes and the same offsets; requests answered to their senders."""
    w = synth.make_workload(4)
    dw = DeviceWorkload(w)
    before = w.ring.reshape(w.n_slots, w.slot_size)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    dw.gather(ctx)
    first = dw.req_arena.cpu().numpy().copy()
    assert np.array_equal(first, w.req_payload)
    offs = dw.req_offsets.cpu().numpy().view(np.uint64)
    assert np.array_equal(offs[:-1], np.concatenate([[0], np.cumsum(w.req_sizes)[:-1]]).astype(np.uint64))
    dw.scatter(ctx)
    after = dw.ring.cpu().numpy().reshape(w.n_slots, w.slot_size)
    used = w.frag_slot
    assert np.array_equal(after[used, 0:6], before[used, 6:12])      # MACs swapped
    assert np.array_equal(after[used, 26:30], before[used, 30:34])    # IPs swapped
    assert np.array_equal(after[used, 58:], before[used, 58:])        # payload echoed
    dw.req_arena.zero_()
    ctx.set_cursor(0, 0)
    dw.gather(ctx)
    assert np.array_equal(dw.req_arena.cpu().numpy(), first)


def test_many_batches_per_call_equal_one_batch_each(ctx):
    """Laying several batches side by side in one call gives every batch the
    bytes it gets alone (what the benchmark's batches-per-launch relies on)."""
    w = synth.make_workload(2, 3)
    one = DeviceWorkload(w)
    many = DeviceWorkload(w, copies=5)
    big = SgContext(0, max_reqs=64, max_frames=1 << 16)
    big.set_cursor(0, 0)
    big.set_cursor(1, 0)
    one.gather(big, rule=True)
    one.scatter(big)
    big.set_cursor(0, 0)
    big.set_cursor(1, 0)
    many.gather(big, rule=True)
    many.scatter(big)
    a = one.req_arena.cpu().numpy()
    b = many.req_arena.cpu().numpy().reshape(5, -1)
    assert all(np.array_equal(a, b[k]) for k in range(5))
    ta = one.tx_ring.cpu().numpy()
    tb = many.tx_ring.cpu().numpy().reshape(5, -1)
    assert all(np.array_equal(ta, tb[k]) for k in range(5))
    big.close()


def test_tiled_request_scan_beyond_8192_requests():
    """More requests than one workgroup scans in two passes: the tiled scan of
    the request totals gives the same offsets as the sequential bump ring."""
    w = synth.make_workload(4, 3000)
    k = 3
    big = SgContext(0, max_reqs=3000 * k, max_frames=1 << 17)
    dw = DeviceWorkload(w, copies=k)
    total = int(w.req_sizes.sum())
    for cursor, cap_extra in ((0, 0), (12345, 777)):
        cap = total * k + cap_extra
        arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
        offs = torch.zeros(dw.n_req + 1, dtype=torch.int64, device=DEV)
        big.set_cursor(0, cursor)
        big.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags,
                         AppRef(arena=arena, cap=cap), offs)
        sizes = np.tile(w.req_sizes, k).astype(np.uint64)
        want = (cursor + np.concatenate([[0], np.cumsum(sizes)])) % cap
        assert np.array_equal(offs.cpu().numpy().view(np.uint64), want.astype(np.uint64))
        assert big.get_cursor(0) == int(want[-1])
        got = arena.cpu().numpy()
        exp = np.zeros(cap, np.uint8)
        pay = np.tile(w.req_payload, k)
        idx = (cursor + np.arange(pay.size, dtype=np.int64)) % cap
        exp[idx] = pay
        assert np.array_equal(got, exp), first_diff(got, exp)
    big.close()


def test_tiled_request_scan_of_70000_small_requests():
    """Seventeen tiles of request totals, many requests of a few dozen bytes:
    same offsets as the sequential bump ring."""
    rng = np.random.default_rng(77)
    n = 70000
    sizes = rng.integers(16, 200, size=n)
    w = synth.make_custom(sizes, [16] * n, order="in_order", seed=5)
    big = SgContext(0, max_reqs=n, max_frames=1 << 17)
    dw = DeviceWorkload(w)
    total = int(w.req_sizes.sum())
    cursor, cap = 4242, total + 999
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    offs = torch.zeros(n + 1, dtype=torch.int64, device=DEV)
    big.set_cursor(0, cursor)
    big.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags,
                     AppRef(arena=arena, cap=cap), offs)
    want = (cursor + np.concatenate([[0], np.cumsum(w.req_sizes.astype(np.uint64))])) % cap
    assert np.array_equal(offs.cpu().numpy().view(np.uint64), want.astype(np.uint64))
    assert big.get_cursor(0) == int(want[-1])
    exp = np.zeros(cap, np.uint8)
    exp[(cursor + np.arange(w.req_payload.size, dtype=np.int64)) % cap] = w.req_payload
    got = arena.cpu().numpy()
    assert np.array_equal(got, exp), first_diff(got, exp)
    big.close()


# ---------------------------------------------------------------- descriptors reused by the echo

def test_echo_scatter_reuses_the_descriptors_of_its_gather(ctx):
    """SG_F_REUSE_DESC: the in-place echo of variable-size requests runs no
    descriptor pass of its own; same bytes, same offsets, same cursor as with
    one.  A call that does not match what was described is refused."""
    w = synth.make_workload(4, 300)
    for reuse in (False, True):
        dw = DeviceWorkload(w, arena_slack=4321)
        start = dw.req_app.cap - 7000
        ctx.set_cursor(0, start)
        ctx.set_cursor(1, start)
        dw.gather(ctx, fixed=False)
        exp, offs, cur = expected_gather(w, arena_cap=dw.req_app.cap, cursor=start)
        assert np.array_equal(dw.req_arena.cpu().numpy(), exp)
        dw.scatter(ctx, fixed=False, reuse=reuse)
        assert getattr(dw, "_described")
        exp_tx, eoffs, ecur = expected_scatter(w, exp, resp_cap=dw.req_app.cap, cursor=start)
        got = dw.ring.cpu().numpy()
        assert np.array_equal(got, exp_tx), f"reuse={reuse}: " + first_diff(got, exp_tx)
        assert np.array_equal(dw.resp_offsets.cpu().numpy().view(np.uint64), eoffs)
        assert ctx.get_cursor(1) == ecur == cur
    # fewer frames than were described: refused, nothing written
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    dw.gather(ctx, fixed=False)
    before = dw.ring.clone()
    a = ctx.scatter_args(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, None, 0, dw.n_req - 1,
                         int(w.resp_first[-2]), w.mtu, dw.resp_app, None, w.flags | capi.F_REUSE_DESC)
    with pytest.raises(SgError) as e:
        ctx.scatter_batch_raw(a)
    assert e.value.code == capi.SG_E_DATA
    assert torch.equal(dw.ring, before)
    # nothing described yet on a fresh context: refused by the host
    fresh = SgContext(0)
    a = ctx.scatter_args(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, None, 0, dw.n_req, dw.n_frames,
                         w.mtu, dw.resp_app, None, w.flags | capi.F_REUSE_DESC)
    with pytest.raises(SgError) as e:
        fresh.scatter_batch_raw(a)
    assert e.value.code == capi.SG_E_INVAL
    fresh.close()


def test_reused_descriptors_are_held_against_the_call_that_uses_them(ctx):
    """SG_F_REUSE_DESC trusts nothing the describing pass did not check: a TX
    ring of smaller slots, another arena, or a smaller mtu than the lengths
    described are refused with SG_E_DATA -- the first two before a byte moves."""
    sizes = [3000, 1400, 4200, 77, 2800, 1401]
    w = synth.make_custom(sizes, sizes, seed=91, in_place=True)
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    dw.gather(ctx, fixed=False)
    assert getattr(dw, "_described")

    def call(tx, mtu, app):
        a = ctx.scatter_args(dw.rx, tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, None, 0, dw.n_req, dw.n_frames,
                             mtu, app, None, w.flags | capi.F_REUSE_DESC)
        with pytest.raises(SgError) as e:
            ctx.scatter_batch_raw(a)
        return e.value

    # a TX ring whose slots are smaller than the slots the lengths were held against
    small = torch.full((w.n_slots * 1024,), 0x5A, dtype=torch.uint8, device=DEV)
    e = call(RingRef(small, w.n_slots, 1024, w.profile), 900, dw.resp_app)
    assert e.code == capi.SG_E_DATA and "longer than a slot" in str(e)
    assert bool((small == 0x5A).all())
    # the same requests, but in another arena than the one the offsets were made for
    other = torch.zeros_like(dw.req_arena)
    tx = torch.full((w.n_slots * w.slot_size,), 0x5A, dtype=torch.uint8, device=DEV)
    e = call(RingRef(tx, w.n_slots, w.slot_size, w.profile), w.mtu, AppRef(arena=other, cap=dw.req_app.cap))
    assert e.code == capi.SG_E_DATA and "destination" in str(e)
    assert bool((tx == 0x5A).all())
    # an arena of another capacity
    e = call(RingRef(tx, w.n_slots, w.slot_size, w.profile), w.mtu, AppRef(arena=dw.req_arena, cap=dw.req_app.cap - 16))
    assert e.code == capi.SG_E_DATA
    assert bool((tx == 0x5A).all())
    # a smaller mtu than the described lengths: the frames beyond it are refused
    e = call(RingRef(tx, w.n_slots, w.slot_size, w.profile), 1000, dw.resp_app)
    assert e.code == capi.SG_E_DATA and "longer than a slot" in str(e)
    # and the matching call still goes through afterwards
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    dw.scatter(ctx, fixed=False, reuse=True)
    exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.req_app.cap)
    assert np.array_equal(dw.ring.cpu().numpy(), exp_tx)


@pytest.mark.parametrize("mode", ["scan", "rule", "one-launch"])
@pytest.mark.parametrize("cfg,n", [(2, 1), (1, 40), (4, 30)])
def test_tables_of_a_small_call_read_from_pinned_host_memory(ctx, cfg, n, mode):
    """The CSR tables of a call (fragment slots, lengths, request and response
    tables, response sizes) left in pinned host memory, where the kernels read
    them across the bus -- what the C++ engine does for calls whose tables the
    calling thread walks: results as with tables in device memory."""
    w = synth.make_workload(cfg, n)
    one_size = bool((w.req_sizes == w.req_sizes[0]).all())
    if mode != "scan" and not one_size:
        pytest.skip("the fragmenting rule needs one request size")
    print(f"case pinned tables cfg={cfg} n={n} mode={mode}", flush=True)
    dw = DeviceWorkload(w)
    pin = lambda t: t.cpu().pin_memory() if t is not None else None
    g = dw.gather_call(ctx, 0, use_frag_len=True, rule=mode != "scan")
    s = dw.scatter_call(ctx, 0, fuse=mode != "scan")
    keep = [pin(dw.frag_slot), pin(dw.frag_len), pin(dw.req_first), pin(dw.tx_slot), pin(dw.hdr_src_slot),
            pin(dw.resp_first), pin(dw.resp_size)]
    g.frag_slot, g.frag_len, g.req_first = keep[0].data_ptr(), keep[1].data_ptr(), keep[2].data_ptr()
    s.tx_slot, s.hdr_src_slot, s.resp_first = keep[3].data_ptr(), keep[4].data_ptr(), keep[5].data_ptr()
    if s.resp_size:
        s.resp_size = keep[6].data_ptr()
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)
    if mode == "one-launch":
        ctx.shunt_batch_raw(g, s)
    else:
        ctx.gather_batch_raw(g)
        ctx.scatter_batch_raw(s)
    exp, eoffs, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    got = dw.req_arena.cpu().numpy()
    assert np.array_equal(got, exp), first_diff(got, exp)
    assert np.array_equal(dw.req_offsets.cpu().numpy().view(np.uint64), eoffs)
    exp_tx, _, _ = expected_scatter(w, exp, resp_cap=dw.resp_app.cap)
    got = dw.tx_ring.cpu().numpy()
    assert np.array_equal(got, exp_tx), first_diff(got, exp_tx)


def test_hardware_queue_of_a_stream(ctx):
    """sg_hip_stream_queue: the same answer for a stream every time it is asked,
    a non-zero one, also for a stream the context does not own; contexts made
    apart from each other sit on different hardware queues where the runtime
    has more than one to give."""
    q1, q2 = ctx.stream_queue(), ctx.stream_queue()
    assert q1 != 0 and q1 == q2
    s = torch.cuda.Stream()
    qs = ctx.stream_queue(s.cuda_stream)
    assert qs != 0 and qs == ctx.stream_queue(s.cuda_stream)
    assert ctx.lib.sg_hip_stream_queue(ctx.h, None, None) == capi.SG_E_INVAL
    others = [ctx]
    for _ in range(2):
        others.append(SgContext.apart_from(others, 0))
    queues = [c.stream_queue() for c in others]
    print("case hardware queues", [hex(q) for q in queues], flush=True)
    assert all(q != 0 for q in queues)
    for c in others[1:]:
        c.close()
    if len(set(queues)) < 2:
        pytest.skip("the runtime gave every stream the same hardware queue (GPU_MAX_HW_QUEUES=1?)")
