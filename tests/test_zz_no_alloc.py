"""The allocation-free gather (sg_hip_gather_batch_static) against the CPU oracle
and against the context's sg_hip_gather_batch on the same inputs, bit for bit,
through the C ABI; that it leaves the device's free memory alone; and that a
call recorded into a HIP graph replays.

Collected last on purpose (the file name sorts behind the other tests): the
static scratch array is shared by every call on the GPU, so these cases also
show that it works after everything else has run.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from splitrpc_amd import capi, synth
from splitrpc_amd.engine import AppRef, DeviceWorkload, SgContext, to_dev

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _static_call(lib, a, cursor, status):
    """One launch-only call on torch's current stream."""
    st = torch.cuda.current_stream().cuda_stream
    return lib.sg_hip_gather_batch_static(0, C.c_void_p(st), C.byref(a),
                                          C.c_void_p(cursor.data_ptr()) if cursor is not None else None,
                                          C.c_void_p(status.data_ptr()) if status is not None else None)


def _both_ways(ctx, w, cap, start, mode, own_words=True):
    """Gathers workload `w` into two arenas of `cap` bytes from bump-ring
    position `start`: through the context and through the allocation-free
    entry point.  Returns what each left behind."""
    dw = DeviceWorkload(w)
    fx = int(w.req_sizes[0]) if mode != "scan" else 0
    flags = capi.F_RULE_FRAGS if mode == "rule" else 0
    out = []
    for static in (False, True):
        arena = torch.full((cap,), 0x5A, dtype=torch.uint8, device=DEV)
        offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
        a = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags,
                            AppRef(arena=arena, cap=cap), offs, flags=flags, fixed_req_size=fx, mtu=w.mtu)
        if not static:
            ctx.set_cursor(0, start)
            ctx.gather_batch_raw(a)
            cur = ctx.get_cursor(0)
            st = 0
        else:
            cursor = torch.tensor([start], dtype=torch.int64, device=DEV)
            status = torch.zeros(1, dtype=torch.int32, device=DEV)
            torch.cuda.synchronize()
            rc = _static_call(ctx.lib, a, cursor if own_words else None, status if own_words else None)
            assert rc == capi.SG_OK, ctx.lib.sg_hip_last_error(None).decode()
            torch.cuda.synchronize()
            cur = int(cursor[0]) if own_words else None
            st = int(status[0])
        out.append((arena.cpu().numpy(), offs.cpu().numpy().view(np.uint64), cur, st))
    return out


@pytest.mark.parametrize("mode", ["scan", "fixed", "rule"])
def test_two_calls_in_a_row_the_second_smaller(mode):
    """The second call leaves most of the scratch the first one filled
    untouched: stale descriptors or totals must not leak into it."""
    ctx = SgContext(0, max_reqs=4096, max_frames=65536)
    rng = np.random.default_rng(5)
    if mode == "scan":
        big = synth.make_custom([int(x) for x in rng.integers(1, 30000, 300)], [64] * 300, seed=21)
        small = synth.make_custom([int(x) for x in rng.integers(1, 9000, 41)], [64] * 41, seed=22)
    else:
        big = synth.make_custom([4200] * 260, [64] * 260, seed=23)
        small = synth.make_custom([4200] * 37, [64] * 37, seed=24)
    cap = int(big.req_sizes.sum()) + 777
    start = cap - 12345  # the ring wraps inside the first call
    for w in (big, small):
        print(f"case no-alloc mode={mode} n_req={w.n_req} n_frags={w.n_frags} start={start}", flush=True)
        (a0, o0, c0, _), (a1, o1, c1, st) = _both_ways(ctx, w, cap, start, mode)
        assert st == 0
        # against the oracle directly: the bytes of the batch where the bump ring puts them, the
        # arena's fill everywhere else, the offsets and the cursor
        exp, eoffs, ecur = oracle.gather(w, arena_cap=cap, cursor=start)
        total = int(w.req_sizes.sum())
        written = np.zeros(cap, bool)
        written[(start + np.arange(total)) % cap] = True
        assert np.array_equal(a1[written], exp[written])
        assert bool((a1[~written] == 0x5A).all())
        assert np.array_equal(o1, eoffs) and c1 == ecur
        # and against the context's call
        assert np.array_equal(o0, o1)
        assert c0 == c1
        assert np.array_equal(a0, a1)
        start = c1
    ctx.close()


def test_cursor_and_status_inside_the_array():
    """cursor == NULL: the array's own word carries over from call to call."""
    ctx = SgContext(0)
    w = synth.make_custom([3000, 1, 5000, 700, 2222, 64], [64] * 6, seed=31)
    dw = DeviceWorkload(w)
    cap = 3 * int(w.req_sizes.sum()) + 100
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    a = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, AppRef(arena=arena, cap=cap),
                        offs)
    torch.cuda.synchronize()
    ends = []
    for call in range(3):
        assert _static_call(ctx.lib, a, None, None) == capi.SG_OK
        torch.cuda.synchronize()
        o = offs.cpu().numpy().view(np.uint64)
        if ends:
            assert int(o[0]) == ends[-1], "the next call starts where the last one ended"
        ends.append(int(o[-1]))
        # the context's call from the same position agrees
        ctx.set_cursor(0, int(o[0]))
        arena2 = torch.zeros(cap, dtype=torch.uint8, device=DEV)
        offs2 = torch.zeros_like(offs)
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, AppRef(arena=arena2, cap=cap),
                         offs2)
        assert np.array_equal(offs2.cpu().numpy().view(np.uint64), o)
        lo, total = int(o[0]), int(w.req_sizes.sum())
        idx = (lo + np.arange(total)) % cap
        assert np.array_equal(arena.cpu().numpy()[idx], arena2.cpu().numpy()[idx])
    ctx.close()


def test_limits_and_refusals():
    ctx = SgContext(0, max_reqs=8192, max_frames=1 << 17)
    w = synth.make_workload(1, 4)
    dw = DeviceWorkload(w)
    a = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, dw.req_app, dw.req_offsets)
    # beyond the array's size: refused by the host with a message, nothing launched
    a.n_frags = capi.STATIC_MAX_FRAMES + 1
    assert _static_call(ctx.lib, a, None, None) == capi.SG_E_INVAL
    assert b"at most" in ctx.lib.sg_hip_last_error(None)
    a.n_frags = dw.n_frags
    a.n_req = capi.STATIC_MAX_REQS + 1
    assert _static_call(ctx.lib, a, None, None) == capi.SG_E_INVAL
    a.n_req = dw.n_req
    assert ctx.lib.sg_hip_gather_batch_static(0, None, None, None, None) == capi.SG_E_INVAL
    # refused by the device: the caller's status word says so and nothing moved
    bad = w.frag_slot.copy()
    bad[3] = w.n_slots + 9
    bad_dev = to_dev(bad, DEV)
    a.frag_slot = bad_dev.data_ptr()
    dw.req_arena.fill_(0xAB)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    cursor = torch.zeros(1, dtype=torch.int64, device=DEV)
    torch.cuda.synchronize()
    assert _static_call(ctx.lib, a, cursor, status) == capi.SG_OK
    torch.cuda.synchronize()
    assert int(status[0]) != 0
    assert bool((dw.req_arena == 0xAB).all())
    assert int(cursor[0]) == 0
    ctx.close()


def test_calls_leave_device_memory_alone_and_replay_from_a_graph():
    """What the entry point exists for: after a warm first call, further calls
    change nothing in the device's free memory, and a call recorded into a HIP
    graph on a stream replays -- twice, with eager work between -- continuing
    the bump ring, like the context's call from the same positions."""
    w = synth.make_custom([4200] * 50, [64] * 50, seed=41)
    dw = DeviceWorkload(w)
    total = int(w.req_sizes.sum())
    cap = 3 * total + 555
    arena = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device=DEV)
    cursor = torch.zeros(1, dtype=torch.int64, device=DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    ctx = SgContext(0)
    for mode in ("rule", "scan"):
        a = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, AppRef(arena=arena, cap=cap),
                            offs, flags=capi.F_RULE_FRAGS if mode == "rule" else 0,
                            fixed_req_size=4200 if mode == "rule" else 0, mtu=w.mtu)
        cursor.zero_()
        torch.cuda.synchronize()
        assert _static_call(ctx.lib, a, cursor, status) == capi.SG_OK  # warm: looks up the array's address
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        for _ in range(5):
            assert _static_call(ctx.lib, a, cursor, status) == capi.SG_OK
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        assert free1 == free0, f"{mode}: free device memory went from {free0} to {free1}"
        assert int(status[0]) == 0
        assert int(cursor[0]) == (6 * total) % cap
        # one call recorded on a side stream, replayed twice
        cursor.zero_()
        s = torch.cuda.Stream()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            rc = ctx.lib.sg_hip_gather_batch_static(0, C.c_void_p(s.cuda_stream), C.byref(a),
                                                    C.c_void_p(cursor.data_ptr()), C.c_void_p(status.data_ptr()))
        assert rc == capi.SG_OK, ctx.lib.sg_hip_last_error(None).decode()
        pos = 0
        for rep in range(2):
            arena.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            exp, eoffs, nxt = oracle.gather(w, arena_cap=cap, cursor=pos)
            got = arena.cpu().numpy()
            assert np.array_equal(got, exp), f"{mode} replay {rep}"
            assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
            assert int(cursor[0]) == nxt and int(status[0]) == 0
            # the context's call from the same position
            ctx.set_cursor(0, pos)
            arena2 = torch.zeros_like(arena)
            a2 = ctx.gather_args(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags,
                                 AppRef(arena=arena2, cap=cap), None, flags=a.flags, fixed_req_size=a.fixed_req_size,
                                 mtu=w.mtu)
            ctx.gather_batch_raw(a2)
            assert torch.equal(arena2, arena) and ctx.get_cursor(0) == nxt
            pos = nxt
            junk = torch.full((1 << 18,), rep, dtype=torch.uint8, device=DEV)
            assert int(junk[3]) == rep
    ctx.close()
