"""The C++ host layer driving the GPU: P2pRpcRRPool + P2pRpcAppRrPool +
P2pRpcSgHipEngine doing one burst of the shunter's work
(src/splitrpc_server/p2p_rpc_dpdk_server.cc:117-189), per request and batched,
against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import oracle
from splitrpc_amd import build, synth

from helpers import conn_templates, first_diff

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def host():
    import torch  # noqa: F401  (loads the HIP runtime the libraries link against)
    h = C.CDLL(build.HOST_LIB)
    h.sgh_serve_gpu.restype = C.c_int64
    h.sgh_serve_gpu.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_uint32,
                                C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint32, C.c_uint32, C.c_int, C.c_int,
                                C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p,
                                C.POINTER(C.c_int)]
    h.sgh_copy_ctx_gpu.argtypes = [C.c_int, C.c_uint64, C.c_uint64, C.c_uint64]
    h.sgh_zc_engine.argtypes = [C.c_uint64]
    h.sgh_window_replay.restype = C.c_int64
    h.sgh_window_replay.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_uint32, C.c_void_p]
    h.sgh_mempool_create.restype = C.c_void_p
    h.sgh_mempool_create.argtypes = [C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_int]
    h.sgh_mempool_destroy.argtypes = [C.c_void_p]
    h.sgh_mempool_mirrored.argtypes = [C.c_void_p]
    for f in ("req_base", "resp_base"):
        getattr(h, "sgh_mempool_" + f).restype = C.c_void_p
        getattr(h, "sgh_mempool_" + f).argtypes = [C.c_void_p]
    for f in ("req_bytes", "resp_bytes"):
        getattr(h, "sgh_mempool_" + f).restype = C.c_uint64
        getattr(h, "sgh_mempool_" + f).argtypes = [C.c_void_p]
    return h


def p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


@pytest.mark.parametrize("per_request", [1, 0, 2, 3, 4],
                         ids=["per-request", "batched", "batched-tx", "tables-pulled", "batched-tx-staged"])
@pytest.mark.parametrize("mirror", [1, 0], ids=["mirrored", "plain"])
@pytest.mark.parametrize("cfg,n,profile", [(1, 12, synth.HDR_BL58), (2, 3, synth.HDR_BL58),
                                           (2, 2, synth.HDR_REF64), (5, 1, synth.HDR_BL58)])
def test_one_burst_of_the_shunter(host, cfg, n, profile, mirror, per_request):
    w = synth.make_workload(cfg, n, profile=profile)
    flags = w.flags & ~synth.F_UDP_CSUM_FULL  # a header-only rewrite cannot see the payload
    if per_request >= 2:
        flags = w.flags                           # the batched TX writes headers with the payload in hand
    print(f"case serve cfg={cfg} n={n} profile={profile} mirror={mirror} per_request={per_request}", flush=True)
    req_size, resp_size = int(w.req_sizes[0]), int(w.resp_sizes[0])
    len_nic = None
    if profile == synth.HDR_REF64:
        len_nic = np.zeros(w.n_slots, np.uint32)
        len_nic[w.frag_slot] = w.frag_len
    tx = w.tx_ring_init.copy()
    req_out = np.zeros(w.n_req * req_size, np.uint8)
    mirrored = C.c_int(-1)
    arr = np.ascontiguousarray(w.arrivals, np.uint32)
    done = host.sgh_serve_gpu(0, p(w.ring), w.n_slots, w.slot_size, profile, p(arr), len(arr), p(len_nic),
                              req_size, resp_size, w.mtu, flags, per_request, mirror, p(w.resp_payload), p(tx),
                              w.tx_n_slots, p(np.ascontiguousarray(w.tx_slot, np.uint32)),
                              p(np.ascontiguousarray(w.hdr_src_slot, np.uint32)), p(req_out), C.byref(mirrored))
    assert done == w.n_req, f"serve returned {done}"
    print("arena mirrored:", mirrored.value, flush=True)
    exp, _, _ = oracle.gather(w)
    assert np.array_equal(req_out, exp), first_diff(req_out, exp)
    exp_tx = w.tx_ring_init.copy()
    if per_request >= 2:
        # fresh response buffers: headers from the connections' templates (rr_set_hdr), the server
        # identity being the one the host layer was started with
        import socket
        import struct
        server = (bytes.fromhex("b8cef6cc6a52"), struct.unpack("!I", socket.inet_aton("192.168.25.1"))[0], 50051)
        # set_conn_info sees the packet of a request that ARRIVES first, whatever its sequence number
        req_of_slot = np.full(w.n_slots, -1, np.int64)
        req_of_slot[w.frag_slot] = np.repeat(np.arange(w.n_req), np.diff(w.req_first.astype(np.int64)))
        first_slots = np.zeros(w.n_req, np.int64)
        for s in arr[::-1]:
            first_slots[req_of_slot[s]] = s
        tm, tk = conn_templates(w, server=server, first_slots=first_slots)
        oracle.scatter(w, w.ring, exp_tx, w.resp_payload, flags=flags, templates=tm, tokens=tk)
    else:
        oracle.scatter(w, w.ring, exp_tx, w.resp_payload, flags=flags)
    assert np.array_equal(tx, exp_tx), first_diff(tx, exp_tx)


def test_copy_context_entry_points_and_small_object_pool(host):
    """CopyCtx + sg_on_gpu_entry + sg_on_gpu (the reference's C entry points)
    move a run; the doorbell sits in a BufItemPool object both sides reach."""
    import torch
    src = torch.arange(5000, dtype=torch.int32, device="cuda").view(torch.uint8)
    dst = torch.zeros(20000 + 64, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    got = host.sgh_copy_ctx_gpu(0, src.data_ptr() + 3, dst.data_ptr() + 7, 19990)
    assert got == 127, f"steps {got:#x}"
    torch.cuda.synchronize()
    assert torch.equal(dst[7:7 + 19990], src[3:3 + 19990])
    assert not bool(dst[:7].any()) and not bool(dst[7 + 19990:].any())


def test_zero_copy_engine_hands_out_the_packet_buffer(host):
    assert host.sgh_zc_engine(0x7f0000001040) == 1


@pytest.mark.parametrize("mode", ["scan", "rule"])
def test_batch_across_the_end_of_a_double_mapped_arena(host, ctx, mode):
    """The request and response arenas of P2pRpcAppRrMemPool are mapped twice
    back to back (the reference's VMM trick, src/p2p_rpc_app_rr.h:60-143), so a
    request that crosses the end of the ring is written and read linearly.
    The oracle wraps byte by byte; both must leave the same bytes."""
    import torch
    from splitrpc_amd import capi
    from splitrpc_amd.engine import AppRef, DeviceWorkload
    from helpers import expected_scatter
    rule = mode == "rule"
    sizes = [70000] * 6 if rule else [70000, 1, 123457, 8, 99999, 70001]
    resp = [50000] * 6 if rule else [1, 50000, 77, 140001, 4200, 1399]
    w = synth.make_custom(sizes, resp, seed=21, flags=synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL)
    dw = DeviceWorkload(w)
    pool = host.sgh_mempool_create(0, 1, 1 << 21, 1 << 21, 1)
    assert pool
    try:
        assert host.sgh_mempool_mirrored(pool) == 1, "HIP virtual memory management is expected on this GPU"
        cap = int(host.sgh_mempool_req_bytes(pool))
        rcap = int(host.sgh_mempool_resp_bytes(pool))
        req_base, resp_base = host.sgh_mempool_req_base(pool), host.sgh_mempool_resp_base(pool)
        assert cap == 1 << 21 and rcap == 1 << 21
        print(f"case mirrored mode={mode} cap={cap}", flush=True)
        app = AppRef(arena_ptr=req_base, cap=cap, mirrored=True)
        rapp = AppRef(arena_ptr=resp_base, cap=rcap, mirrored=True)
        stage = torch.zeros(cap, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()   # the context launches on its own stream
        ctx.copy_runs([stage.data_ptr()], [req_base], [cap])           # clear the arena
        start = cap - 100000                                           # the second request crosses the end
        ctx.set_cursor(0, start)
        offs = torch.zeros(w.n_req + 1, dtype=torch.int64, device="cuda")
        ctx.gather_batch(dw.rx, dw.frag_slot, None, dw.req_first, dw.n_req, dw.n_frags, app, offs,
                         flags=capi.F_RULE_FRAGS if rule else 0, fixed_req_size=sizes[0] if rule else 0, mtu=w.mtu)
        exp, eoffs, ecur = oracle.gather(w, arena_cap=cap, cursor=start)
        ctx.copy_runs([req_base], [stage.data_ptr()], [cap])
        got = stage.cpu().numpy()
        assert np.array_equal(got, exp), first_diff(got, exp)
        assert np.array_equal(offs.cpu().numpy().view(np.uint64), eoffs)
        assert ctx.get_cursor(0) == ecur
        # the second mapping shows the same bytes
        ctx.copy_runs([req_base + cap], [stage.data_ptr()], [cap])
        assert np.array_equal(stage.cpu().numpy(), exp)

        # responses: lay them out in the response arena the way the oracle's bump ring does
        rstart = rcap - 60000
        resp_arena = np.zeros(rcap, np.uint8)
        pos = rstart
        for r in range(w.n_req):
            n = int(w.resp_sizes[r])
            src = w.resp_payload[sum(int(x) for x in w.resp_sizes[:r]):][:n]
            idx = (pos + np.arange(n)) % rcap
            resp_arena[idx] = src
            pos = (pos + n) % rcap
        stage.copy_(torch.from_numpy(resp_arena).cuda())
        torch.cuda.synchronize()
        ctx.copy_runs([stage.data_ptr()], [resp_base], [rcap])
        ctx.set_cursor(1, rstart)
        sz = None if rule else dw.resp_size
        ctx.scatter_batch(dw.rx, dw.tx, dw.tx_slot, dw.hdr_src_slot, dw.resp_first, sz, resp[0] if rule else 0,
                          dw.n_req, dw.n_frames, w.mtu, rapp, None, w.flags)
        tx = w.tx_ring_init.copy()
        oracle.scatter(w, w.ring, tx, resp_arena, arena_cap=rcap, cursor=rstart,
                       fixed_size=resp[0] if rule else None)
        got = dw.tx_ring.cpu().numpy()
        assert np.array_equal(got, tx), first_diff(got, tx)
    finally:
        host.sgh_mempool_destroy(pool)


def test_batching_window_over_the_slot_ring(host):
    """SgBatchWindow (the window of dynamic_batching_sync_worker_loop,
    src/p2p_rpc_async_app_server.h:220-263) against a list simulation: windows
    are runs of consecutive RX_COMPLETE slots from the consumer index, capped
    at max_batch, wrapping around the ring."""
    rng = np.random.default_rng(4)
    pool_size = 11
    ops, sim_state, pi, ci, want = [], [0] * pool_size, 0, 0, []
    for _ in range(400):
        free = sum(1 for x in sim_state if x == 0)
        if rng.random() < 0.5 and free:
            k = int(rng.integers(1, free + 1))
            ops.append(k)
            for _ in range(k):
                assert sim_state[pi] == 0
                sim_state[pi] = 1
                pi = (pi + 1) % pool_size
        else:
            m = int(rng.integers(1, 9))
            ops.append(-m)
            start, n = ci, 0
            while n < m and n < pool_size and sim_state[ci] == 1:
                sim_state[ci] = 0
                ci = (ci + 1) % pool_size
                n += 1
            want.append((start, n))
    ops_a = np.array(ops, np.int32)
    out = np.zeros(2 * len(ops), np.int32)
    n = host.sgh_window_replay(0, pool_size, p(ops_a), len(ops_a), p(out))
    assert n == len(want)
    got = [(int(out[2 * i]), int(out[2 * i + 1])) for i in range(n)]
    assert got == want
    assert max(g[1] for g in got) > 1 and any(g[1] == 0 for g in got)
