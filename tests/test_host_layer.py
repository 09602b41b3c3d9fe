"""The C++ host layer (splitrpc_amd/host/*.h: the reference's P2pRpcRr /
P2pRpcRRPool / P2pRpcTring / gather_skbs interfaces) through its C shim,
against the CPU oracle and the compiled reference headers.  No GPU needed."""
import ctypes as C
import os

import numpy as np
import pytest

import oracle
from splitrpc_amd import build, synth

L = oracle.lib()
REF = oracle.ref()


@pytest.fixture(scope="module")
def host():
    assert os.path.exists(build.HOST_LIB), "build first: python -m splitrpc_amd.build"
    h = C.CDLL(build.HOST_LIB)
    h.sgh_layout.restype = C.c_uint64
    h.sgh_skbs.restype = C.c_uint64
    h.sgh_skbs.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p]
    h.sgh_tring_replay.argtypes = [C.c_uint64, C.c_uint64, C.c_void_p, C.c_uint32, C.c_void_p]
    h.sgh_pool_replay.restype = C.c_int64
    h.sgh_pool_replay.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64, C.c_void_p, C.c_uint32,
                                  C.c_void_p, C.c_uint64, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_void_p]
    h.sgh_pool_exhaust.restype = C.c_uint64
    h.sgh_pool_exhaust.argtypes = [C.c_int, C.c_uint32]
    h.sgh_ring_stress.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32]
    return h


def p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def test_layouts(host):
    want = [8194, 16386, 24576, 16, 128, 14, 20, 8, 42, 1024, 8192, 8192, 16384, 8192, 16384, 24568, 8, 32, 64, 96,
            2, 10, 12, 16, 4, 6, 9]
    got = [host.sgh_layout(i) for i in range(27)]
    assert got == want
    if REF is not None:  # the numbers above are the compiled reference's
        assert got == [REF.ref_layout(i) for i in range(27)]
    # p2p_rpc_hdr: 64 bytes, token @42, sock_perf_header @50, seq_num @58 (src/p2p_rpc.h:10-17)
    assert [host.sgh_layout(i) for i in range(27, 31)] == [64, 42, 50, 58]


def test_run_table_builders_match_the_oracle(host):
    rng = np.random.default_rng(31)
    for trial in range(300):
        n = int(rng.integers(0, 60)) if trial else 0
        m = max(n, 1)
        sizes = rng.integers(1, 3000, m).astype(np.uint64)
        ptrs = np.zeros(m, np.uint64)
        cur = 1 << 22
        for i in range(m):
            if i and rng.random() < 0.5:
                cur = int(ptrs[i - 1] + sizes[i - 1])
            else:
                cur += int(rng.integers(4000, 9000))
            ptrs[i] = cur
        for scatter in (0, 1):
            io, oo, lo = np.zeros(1024, np.uint64), np.zeros(1024, np.uint64), np.zeros(1024, np.uint64)
            k = host.sgh_skbs(scatter, p(ptrs), p(sizes), n, 0x5000, p(io), p(oo), p(lo))
            b, skb = oracle.Bufs(), oracle.SkBuf()
            for i in range(m):
                b.burst_items[i], b.item_size[i] = int(ptrs[i]), int(sizes[i])
            b.num_items = n
            (L.sgo_scatter_skbs if scatter else L.sgo_gather_skbs)(C.byref(skb), C.byref(b), 0x5000)
            assert k == skb.num_items
            assert io[:k].tolist() == [skb.i_buf[i] for i in range(k)]
            assert oo[:k].tolist() == [skb.o_buf[i] for i in range(k)]
            assert lo[:k].tolist() == [skb.len[i] for i in range(k)]


def test_tring(host):
    rng = np.random.default_rng(32)
    sizes = rng.integers(1, 5000, 300).astype(np.uint64)
    out = np.zeros(300, np.uint64)
    host.sgh_tring_replay(1 << 32, 77777, p(sizes), 300, p(out))
    t = oracle.Tring()
    L.sgo_tring_init(C.byref(t), 1 << 32, 77777)
    assert out.tolist() == [L.sgo_tring_get_next(C.byref(t), int(s)) for s in sizes]
    if REF is not None:
        ref_out = np.zeros(300, np.uint64)
        REF.ref_tring_replay(1 << 32, 77777, p(sizes), 300, p(ref_out))
        assert np.array_equal(out, ref_out)


def _pool_replay(host, w, arrivals, len_nic=None, req_size=0, pool_size=-1):
    n = len(arrivals)
    fs, fl = np.zeros(n + 1, np.uint32), np.zeros(n + 1, np.uint32)
    rf, tok = np.zeros(n + 2, np.uint32), np.zeros(n + 1, np.uint64)
    left = np.zeros(1, np.uint64)
    arr = np.ascontiguousarray(arrivals, dtype=np.uint32)
    done = host.sgh_pool_replay(p(w.ring), w.n_slots, w.slot_size, w.profile, 0x7F0000000000, p(arr), n,
                                p(len_nic), req_size, pool_size, p(fs), p(fl), p(rf), p(tok), p(left))
    assert done >= 0
    nf = int(rf[done])
    return fs[:nf], fl[:nf], rf[:done + 1], tok[:done], int(left[0])


@pytest.mark.parametrize("cfg,n", [(1, 10), (2, 2), (3, 50), (4, 80), (5, 2)])
def test_pool_reassembly_matches_the_oracle(host, cfg, n):
    w = synth.make_workload(cfg, n)
    got = _pool_replay(host, w, w.arrivals)
    want = oracle.reassemble(w)
    for g, e in zip(got[:4], want):
        assert np.array_equal(g, e)
    assert got[4] == 0
    # and with the arrivals shuffled
    arr = np.random.default_rng(cfg).permutation(w.arrivals)
    got = _pool_replay(host, w, arr)
    want = oracle.reassemble(w, arrivals=arr)
    for g, e in zip(got[:4], want):
        assert np.array_equal(g, e)


def test_pool_reassembly_ref64_by_request_size(host):
    """The reference's own readiness rule: payload_size == max_payload_size."""
    w = synth.make_workload(2, 3, profile=synth.HDR_REF64)
    len_nic = np.zeros(w.n_slots, np.uint32)
    len_nic[w.frag_slot] = w.frag_len
    size = int(w.req_sizes[0])
    got = _pool_replay(host, w, w.arrivals, len_nic=len_nic, req_size=size)
    want = oracle.reassemble(w, req_size=size, frag_len_nic=len_nic)
    for g, e in zip(got[:4], want):
        assert np.array_equal(g, e)
    assert np.array_equal(got[0], w.frag_slot)


def test_lost_fragment_parks_the_request(host):
    """A lost fragment leaves its request in the cache for good
    (src/p2p_rpc_rr_pool_ng.h:57-64): nothing is handed over for it."""
    w = synth.make_workload(1, 6)
    arr = np.delete(w.arrivals, 4)
    fs, fl, rf, tok, left = _pool_replay(host, w, arr)
    assert len(tok) == 5 and left == 1


def test_pool_grows_when_exhausted(host):
    assert host.sgh_pool_exhaust(4, 3) == 3      # pool_size - 1 rrs, all taken
    assert host.sgh_pool_exhaust(4, 10) == 10    # seven more were allocated


def test_pointer_ring_multi_producer_multi_consumer(host):
    assert host.sgh_ring_stress(4, 20000, 64) == 1
    assert host.sgh_ring_stress(2, 1000, 2) == 1


# ---------------------------------------------------------------- client patterns (load generator)

@pytest.mark.parametrize("slot_size", [2048, 9216, 1536, 4096])
@pytest.mark.parametrize("profile", [0, 1])
def test_slot_of_a_payload_pointer_by_shift_and_by_division(host, slot_size, profile):
    """The batched calls turn payload pointers into slot indices with a shift
    where slots are a power of two bytes and a division elsewhere: both forms
    against the arithmetic, on payload starts, pointers off a payload start
    and pointers outside the ring."""
    host.sgh_slots_of_payloads.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_uint32,
                                           C.c_void_p, C.c_void_p]
    host.sgh_slots_of_payloads.restype = None
    rng = np.random.default_rng(slot_size + profile)
    base, n_slots, hl = 0x7F0000001000 + 2 * int(rng.integers(0, 64)), 777, 64 if profile else 58
    slots = rng.integers(0, n_slots, 4000)
    good = base + slots * slot_size + hl
    off = good + rng.integers(1, slot_size, 4000)                     # inside a slot, not at its payload
    outside = np.concatenate([base + (n_slots + rng.integers(0, 9, 50)) * slot_size + hl,      # behind the ring
                              base - rng.integers(1, 5, 50) * slot_size + hl,                  # in front of it
                              np.array([base, base + hl - 1, 0], np.int64)])
    p = np.ascontiguousarray(np.concatenate([good, off, outside]).astype(np.uint64))
    want = np.concatenate([slots, np.full(off.size + outside.size, -1)]).astype(np.int64)
    by_walk, by_div = np.zeros(p.size, np.int64), np.zeros(p.size, np.int64)
    pv = lambda x: x.ctypes.data_as(C.c_void_p)
    host.sgh_slots_of_payloads(base, n_slots, slot_size, profile, pv(p), p.size, pv(by_walk), pv(by_div))
    assert np.array_equal(by_div, want)
    assert np.array_equal(by_walk, want)


def test_state_word_wait_is_bounded(host):
    """AppRrRunNotify waits on the calling thread: the word has to be set by
    somebody else.  Another thread setting it ends the wait; nobody setting it
    in time ends it too, with a false return and a count."""
    host.sgh_notify_wait.argtypes = [C.c_uint32, C.c_uint64]
    assert host.sgh_notify_wait(2000, 2_000_000_000) == 1 | 4        # set after 2 ms: seen
    assert host.sgh_notify_wait(200_000, 20_000_000) == 2 | 4        # set after 200 ms, bound 20 ms: gave up
    assert host.sgh_notify_wait(0, 0) & 1                            # no bound: still returns once set


def test_bench_has_measured_traffic_for_every_default_call():
    """roofline.traffic comes from counter runs of the default calls: a default
    that changes without a fresh counter run would silently report None."""
    import bench
    for cfg, bpl in bench.DEFAULT_BPL.items():
        for kernel in ("k_gather", "k_scatter"):
            assert (cfg, bpl, kernel) in bench.MEASURED_TRAFFIC, (cfg, bpl, kernel)
            assert bench.MEASURED_TRAFFIC[(cfg, bpl, kernel)] > 0


def test_measured_traffic_belongs_to_the_kernel_sources_in_the_tree():
    """The traffic figures are counter readings of particular kernels: after a
    change to the kernel sources they have to be taken again (the commands
    head profiles/copy_kernels_all_workloads_traffic_time_instructions.txt),
    and bench.MEASURED_TRAFFIC / TRAFFIC_MEASURED_WITH updated with them.
    Until then the bench line reports `traffic` as null."""
    import bench
    assert bench.traffic_is_current(), "kernel sources changed since roofline.traffic was measured"


def test_client_patterns_and_checks_through_the_cpu_path():
    """The reference clients' request patterns and reply checks
    (lib_loadgen/echo_client.cc, vec_add_client.cc) around the oracle's gather
    and scatter: what the echo client gets back passes its own check, a
    flipped byte does not."""
    import oracle
    from splitrpc_amd import loadgen, synth
    assert bytes(loadgen.create_echo_request(8193)[[0, 1, 8191, 8192]]) == bytes([0xDE, 2, 2, 0xAD])
    assert bytes(loadgen.create_vec_add_request(6)) == bytes([0xDE, 0xAD, 0xBE, 0xEF, 0xDE, 0xAD])
    assert loadgen.complete_echo_reply(loadgen.create_echo_request(20000), 20000) == 0
    assert loadgen.complete_echo_reply(loadgen.create_echo_request(20000), 20001) == 1
    assert loadgen.complete_vec_add_reply(loadgen.create_vec_add_request(64) + 1, 64) == 0
    assert loadgen.complete_vec_add_reply(loadgen.create_vec_add_request(64), 64) == 1

    w = loadgen.client_workload("echo", 5, 20000)
    assert w.profile == synth.HDR_REF64 and w.tx_in_place
    arena, _, _ = oracle.gather(w, use_frag_len=True)
    ring = w.ring.copy()
    oracle.scatter(w, ring, ring, arena)
    assert loadgen.verify_responses(w, ring, "echo") == 0
    ring[int(w.tx_slot[3]) * w.slot_size + 64 + 7] ^= 1
    assert loadgen.verify_responses(w, ring, "echo") == 1

    w = loadgen.client_workload("vec_add", 4, 5000, resp_size=3000)
    arena, _, _ = oracle.gather(w, use_frag_len=True)
    served = (arena.reshape(4, 5000)[:, :3000].astype(np.uint16) + 1).astype(np.uint8).reshape(-1)  # the model
    tx = w.tx_ring_init.copy()
    oracle.scatter(w, w.ring, tx, served)
    assert loadgen.verify_responses(w, tx, "vec_add") == 0


# ---------------------------------------------------------------- sanitizers on the host layer

@pytest.mark.parametrize("san", ["thread", "address,undefined"])
def test_rings_and_pool_under_sanitizers(san, tmp_path):
    """The request pool and its rings between a receive and a shunter thread,
    built with the thread sanitizer and with the address + undefined-behaviour
    sanitizers (host code only: tests/host_sanitize.cpp)."""
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++")
    exe = str(tmp_path / "host_sanitize")
    cmd = [gxx, "-std=c++17", "-O1", "-g", f"-fsanitize={san}", "-fno-sanitize-recover=all",
           "-I", os.path.join(root, "splitrpc_amd", "host"), "-I", os.path.join(root, "include"),
           os.path.join(root, "tests", "host_sanitize.cpp"), "-o", exe, "-lpthread"]
    built = subprocess.run(cmd, capture_output=True, text=True)
    if built.returncode != 0 and "sanitize" in built.stderr and "cannot find" in built.stderr:
        pytest.skip("sanitizer runtime not installed")
    assert built.returncode == 0, built.stderr[-2000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, (run.stdout + run.stderr)[-3000:]
    assert "host sanitize: ok" in run.stdout
