"""The C++ host layer driving the GPU: P2pRpcRRPool + P2pRpcAppRrPool +
P2pRpcSgHipEngine doing one burst of the shunter's work
(src/splitrpc_server/p2p_rpc_dpdk_server.cc:117-189), per request and batched,
against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import oracle
from splitrpc_amd import build, synth

from helpers import first_diff

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
    return h


def p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


@pytest.mark.parametrize("per_request", [1, 0], ids=["per-request", "batched"])
@pytest.mark.parametrize("mirror", [1, 0], ids=["mirrored", "plain"])
@pytest.mark.parametrize("cfg,n,profile", [(1, 12, synth.HDR_BL58), (2, 3, synth.HDR_BL58),
                                           (2, 2, synth.HDR_REF64), (5, 1, synth.HDR_BL58)])
def test_one_burst_of_the_shunter(host, cfg, n, profile, mirror, per_request):
    w = synth.make_workload(cfg, n, profile=profile)
    flags = w.flags & ~synth.F_UDP_CSUM_FULL  # a header-only rewrite cannot see the payload
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
    oracle.scatter(w, w.ring, exp_tx, w.resp_payload, flags=flags)
    assert np.array_equal(tx, exp_tx), first_diff(tx, exp_tx)
