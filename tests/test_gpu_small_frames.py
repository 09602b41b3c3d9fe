"""Short frames and fragments, several to a wavefront (k_gather_small,
k_scatter_small): every layout and flag the one-wavefront-per-frame kernels
handle, held against the oracle with the short-frame path forced, left to the
library's own choice, and switched off."""
import numpy as np
import pytest
import torch

import oracle
from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, SgContext, to_dev

from helpers import conn_templates, expected_gather, expected_scatter, first_diff

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PATHS = {"forced": capi.F_FORCE_SMALL, "auto": 0, "off": capi.F_NO_SMALL}


def _check(ctx, w, extra, cap_slack=0, cursor=0, templates=False):
    dw = DeviceWorkload(w, arena_slack=cap_slack)
    ctx.set_cursor(0, cursor)
    ctx.set_cursor(1, 0)
    dw.req_arena.zero_() if not w.in_tensor_sizes else None
    dw.gather(ctx, flags=extra, rule=True, use_frag_len=w.profile == synth.HDR_REF64)
    if w.in_tensor_sizes:
        exp, _, _ = expected_gather(w)
        for t, e in zip(dw.in_tensors, exp):
            got = t.cpu().numpy()
            assert np.array_equal(got, e), first_diff(got, e)
        gathered = None
    else:
        exp, offs, _ = expected_gather(w, arena_cap=dw.req_app.cap, cursor=cursor)
        got = dw.req_arena.cpu().numpy()
        assert np.array_equal(got, exp), first_diff(got, exp)
        assert np.array_equal(dw.req_offsets.cpu().numpy().view(np.uint64), offs)
        gathered = exp
    tm = tk = None
    if templates:
        tm, tk = conn_templates(w, seed=3)
    dw.scatter(ctx, flags=extra, templates=to_dev(tm.reshape(-1), DEV) if templates else None,
               tokens=to_dev(tk, DEV) if templates else None)
    exp_tx, _, _ = expected_scatter(w, gathered, templates=tm, tokens=tk)
    got = dw.tx_ring.cpu().numpy()
    assert np.array_equal(got, exp_tx), first_diff(got, exp_tx)


@pytest.mark.parametrize("path", list(PATHS))
@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64], ids=["bl58", "ref64"])
@pytest.mark.parametrize("last", [1, 15, 16, 17, 100, 127, 128, 129, 239, 240, 479, 480, 481, 700, 991, 992, 993, 1399])
def test_remainder_fragment_of_every_length(ctx, last, profile, path):
    """Requests and responses of two full frames plus a remainder of `last`
    bytes: 16 lanes up to 480 bytes (8 in the scatter up to 128), 32 up to 992,
    a wavefront beyond."""
    size = 2 * 1400 + last
    w = synth.make_custom([size] * 11, [size] * 11, seed=last, profile=profile,
                          flags=synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL)
    print(f"case small last={last} profile={profile} path={path}", flush=True)
    _check(ctx, w, PATHS[path], cap_slack=333, cursor=w.n_req * size + 333 - 4000)


@pytest.mark.parametrize("path", ["auto", "off"])
@pytest.mark.parametrize("flags", [0, 2, 2 | 8, 1, 4, 1 | 4, 7, 15])
@pytest.mark.parametrize("size,mtu", [(40, 1400), (1, 64), (300, 64), (480, 480), (992, 992), (3000, 200), (3136, 448)])
def test_calls_made_of_short_frames_only(ctx, size, mtu, flags, path):
    """Frames no longer than 992 bytes: the whole call goes several frames to a
    wavefront (the LeNet responses of 40 bytes among them)."""
    w = synth.make_custom([size] * 37, [size] * 37, mtu=mtu, seed=size + mtu, flags=flags)
    _check(ctx, w, PATHS[path])


@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64], ids=["bl58", "ref64"])
@pytest.mark.parametrize("flags", [0, synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL])
def test_single_frame_responses_of_every_small_size(ctx, profile, flags):
    """Requests and responses of one short frame, eight to a wavefront up to
    128 bytes and four beyond: every size class and every phase (payloads packed
    back to back start at all offsets modulo 16), edge bytes on both sides of
    the aligned chunks included."""
    for size in list(range(1, 50)) + list(range(50, 260, 7)) + [127, 128, 129, 130]:
        w = synth.make_custom([size] * 19, [size] * 19, seed=1000 + size, profile=profile, flags=flags)
        print(f"case single short frame size={size} profile={profile} flags={flags}", flush=True)
        _check(ctx, w, 0, cap_slack=77, cursor=5)


@pytest.mark.parametrize("path", list(PATHS))
def test_headers_from_templates_on_short_frames(ctx, path):
    for profile in (synth.HDR_BL58, synth.HDR_REF64):
        w = synth.make_custom([3072] * 9, [3072] * 9, seed=5, profile=profile, flags=synth.F_UDP_CSUM_PSEUDO | synth.F_REF_QUIRKS)
        _check(ctx, w, PATHS[path], templates=True)
        w = synth.make_custom([100] * 9, [100] * 9, seed=6, profile=profile, flags=synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL)
        _check(ctx, w, PATHS[path], templates=True)


@pytest.mark.parametrize("path", list(PATHS))
def test_tensor_major_buffers_and_the_fragment_between_two_tensors(ctx, path):
    """Workload 3's shape: the first fragment runs from the ids tensor into the
    mask tensor (two runs in flight), the remainder is a short fragment; the
    responses end in a short frame too."""
    w = synth.make_workload(3, 77)
    _check(ctx, w, PATHS[path])
    # a short fragment that itself straddles two tensors goes byte by byte
    w = synth.make_custom([1400 + 600] * 13, [200] * 13, seed=8, in_tensor_sizes=[1700, 300])
    _check(ctx, w, PATHS[path])
    w = synth.make_custom([500] * 13, [500] * 13, seed=9, in_tensor_sizes=[123, 377], out_tensor_sizes=[500])
    _check(ctx, w, PATHS[path])


def test_counts_on_the_device_with_short_frames(ctx):
    """Fewer requests than the launch was sized for: the short-frame kernels stop
    where the device-resident count says."""
    w = synth.make_custom([3000] * 20, [3000] * 20, seed=12, flags=synth.F_UDP_CSUM_PSEUDO)
    dw = DeviceWorkload(w)
    for live in (0, 1, 7, 20):
        counts = to_dev(np.array([live, live * 3, 0, 0], np.uint32), DEV)
        ctx.set_cursor(0, 0)
        ctx.set_cursor(1, 0)
        dw.req_arena.fill_(0xEE)
        dw.tx_ring.copy_(torch.from_numpy(w.tx_ring_init).to(DEV))
        ga = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app, None,
                             flags=capi.F_RULE_FRAGS | capi.F_FORCE_SMALL, fixed_req_size=3000, mtu=w.mtu, counts=counts)
        ctx.gather_batch_raw(ga)
        exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
        want = np.full(dw.req_app.cap, 0xEE, np.uint8)
        want[:live * 3000] = exp[:live * 3000]
        got = dw.req_arena.cpu().numpy()
        assert np.array_equal(got, want), f"live={live}: " + first_diff(got, want)
        assert ctx.get_cursor(0) == (live * 3000) % dw.req_app.cap
        sa = ctx.scatter_args(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, None, 3000, dw.n_req,
                              dw.n_frames, w.mtu, dw.resp_app, None, w.flags | capi.F_FORCE_SMALL, counts=counts)
        ctx.scatter_batch_raw(sa)
        exp_tx, _, _ = expected_scatter(w, exp)
        per = w.slot_size
        want_tx = w.tx_ring_init.copy().reshape(-1, per)
        served = w.tx_slot[:live * 3]
        want_tx[served] = exp_tx.reshape(-1, per)[served]
        got = dw.tx_ring.cpu().numpy()
        assert np.array_equal(got, want_tx.reshape(-1)), f"live={live}: " + first_diff(got, want_tx.reshape(-1))
