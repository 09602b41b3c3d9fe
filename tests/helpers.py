"""Shared pieces of the parity tests: run the CPU oracle on a workload and
return what the HIP path has to reproduce bit for bit."""
import numpy as np

import oracle


def expected_gather(w, arena_cap=None, cursor=0):
    return oracle.gather(w, arena_cap=arena_cap, cursor=cursor)


def expected_scatter(w, gathered, resp_cap=None, cursor=0, flags=None):
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
    offs, cur = oracle.scatter(w, rx, tx, src, arena_cap=cap, cursor=cursor, flags=flags)
    return tx, offs, cur


def first_diff(a: np.ndarray, b: np.ndarray) -> str:
    if a.shape != b.shape:
        return f"shape {a.shape} vs {b.shape}"
    idx = np.flatnonzero(a != b)
    if idx.size == 0:
        return "equal"
    i = int(idx[0])
    return f"{idx.size} bytes differ, first at {i}: got {a[i]} want {b[i]}"
