"""Writes tests/golden/digests.json: SHA-256 digests of what the CPU oracle
produces for seeded, scaled-down rings of the five workloads (gathered bytes,
offsets, response packets).  Run it in the container that holds the reference
tree, after tests/test_oracle_pins.py passes there (those tests pin the oracle
against the compiled reference headers); the digests then keep the oracle from
drifting on machines that have no reference tree.

    python -m tests.golden.make_golden
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CASES = [(1, 6), (2, 2), (3, 12), (4, 40), (5, 1)]


def _sha(*arrays) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def digests() -> dict:
    import oracle
    from splitrpc_amd import synth
    out = {}
    for cfg, n in CASES:
        w = synth.make_workload(cfg, n)
        g, offs, cur = oracle.gather(w)
        key = f"{w.name}-{n}"
        if w.in_tensor_sizes:
            out[key + "-gather"] = _sha(*g)
        else:
            out[key + "-gather"] = _sha(g, offs)
        if w.tx_in_place:
            tx = w.ring.copy()
            oracle.scatter(w, tx, tx, g)
        else:
            tx = w.tx_ring_init.copy()
            src = [w.resp_payload.copy()] if w.out_tensor_sizes else w.resp_payload
            oracle.scatter(w, w.ring, tx, src)
        out[key + "-scatter"] = _sha(tx)
        out[key + "-ring"] = _sha(w.ring, w.frag_slot, w.frag_len, w.req_first)
    return out


if __name__ == "__main__":
    d = digests()
    with open(os.path.join(HERE, "digests.json"), "w") as f:
        json.dump(d, f, indent=1, sort_keys=True)
    print("wrote", len(d), "digests")
