"""Shared pieces of the parity tests: run the CPU oracle on a workload and
return what the HIP path has to reproduce bit for bit."""
import numpy as np

import oracle


def expected_gather(w, arena_cap=None, cursor=0):
    return oracle.gather(w, arena_cap=arena_cap, cursor=cursor)


def expected_scatter(w, gathered, resp_cap=None, cursor=0, flags=None, templates=None, tokens=None):
    """Returns the TX ring bytes after the oracle's scatter (+ offsets, cursor)."""
    if w.tx_in_place:
        tx = w.ring.copy()
        rx = tx
        src = gathered
        cap = gathered.size if resp_cap is None else resp_cap
    else:
        tx = w.tx_ring_init.copy()
        rx = w.ring
        if w.out_tensor_sizes:
            per = int(sum(w.out_tensor_sizes))
            rp = w.resp_payload.reshape(w.n_req, per)
            src, o = [], 0
            for s in w.out_tensor_sizes:
                src.append(np.ascontiguousarray(rp[:, o:o + s]).reshape(-1))
                o += s
            cap = None
        else:
            src = w.resp_payload if w.resp_payload.size >= 16 else np.concatenate(
                [w.resp_payload, np.zeros(16 - w.resp_payload.size, np.uint8)])
            cap = max(int(w.resp_payload.size), 16) if resp_cap is None else resp_cap
    offs, cur = oracle.scatter(w, rx, tx, src, arena_cap=cap, cursor=cursor, flags=flags,
                              templates=templates, tokens=tokens)
    return tx, offs, cur


def first_diff(a: np.ndarray, b: np.ndarray) -> str:
    if a.shape != b.shape:
        return f"shape {a.shape} vs {b.shape}"
    idx = np.flatnonzero(a != b)
    if idx.size == 0:
        return "equal"
    i = int(idx[0])
    return f"{idx.size} bytes differ, first at {i}: got {a[i]} want {b[i]}"


def conn_templates(w, seed=0, server=None, first_slots=None):
    """Per-request connection templates the way the reference builds them: a
    server-side template (gen_*_header_template) pointed at the client by
    set_conn_info with the request's first packet.  Returns (n_req x 64 uint8,
    n_req uint64 tokens read from those packets).  ``server`` = (mac bytes,
    ip, port) fixes the server's identity as initialize_src_conn_info does
    (src/p2p_rpc_conn_info.h:50-70: both MACs the server's, destination
    0.0.0.0:0); otherwise identities are random.  ``first_slots[r]`` names the
    packet of request r that reached the server first (the one set_conn_info
    sees); default: fragment 0."""
    import ctypes as C
    L = oracle.lib()
    rng = np.random.default_rng(seed)
    pp = lambda a: a.ctypes.data_as(C.c_void_p)
    tm = np.zeros((w.n_req, 64), np.uint8)
    tk = np.zeros(w.n_req, np.uint64)
    for r in range(w.n_req):
        if w.req_first[r + 1] == w.req_first[r]:
            continue
        slot = int(first_slots[r]) if first_slots is not None else int(w.frag_slot[w.req_first[r]])
        recv = np.ascontiguousarray(w.ring[slot * w.slot_size: slot * w.slot_size + 64])
        t = np.zeros(64, np.uint8)
        if server is not None:
            sm = dm = np.frombuffer(bytes(server[0]), np.uint8).copy()
            L.sgo_gen_hdr_template(pp(t), pp(sm), pp(dm), int(server[1]), 0, int(server[2]), 0)
        else:
            sm, dm = rng.integers(0, 256, 6, dtype=np.uint8), rng.integers(0, 256, 6, dtype=np.uint8)
            L.sgo_gen_hdr_template(pp(t), pp(sm), pp(dm), int(rng.integers(0, 2 ** 32)), int(rng.integers(0, 2 ** 32)),
                                   int(rng.integers(0, 65536)), int(rng.integers(0, 65536)))
        L.sgo_set_conn_info(pp(t), pp(recv), w.profile)
        tm[r] = t
        tk[r] = recv[42:50].view(np.uint64)[0]
    return tm, tk
