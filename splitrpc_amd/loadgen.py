"""Client-side request patterns and reply checks of the reference's load
generator, for host-only replay: rings of requests a server built on this
library can be fed with, and the verification the clients run on what comes
back.

  echo     src/lib_loadgen/echo_client.cc:7-66: DE AD BE EF cycling at every
           8192nd byte, 2 everywhere else; the reply must be the request
  vec_add  src/lib_loadgen/vec_add_client.cc:7-35: MAGIC[i % 4]; the reply
           must be MAGIC[i % 4] + 1

``client_workload`` lays such requests out in a ring with the reference's own
64-byte headers (or the 58-byte benchmark headers) the way the NIC would have
left them, with the tables of the receive path beside them (see
``splitrpc_amd.synth``).
"""
from __future__ import annotations

from typing import Optional

import numpy as np

from . import synth

MAGIC_STRING = np.array([0xDE, 0xAD, 0xBE, 0xEF], dtype=np.uint8)


def create_echo_request(size: int) -> np.ndarray:
    """CreateEchoRequest, echo_client.cc:11-24."""
    req = np.full(size, 2, dtype=np.uint8)
    marks = np.arange(0, size, 8192)
    req[marks] = MAGIC_STRING[np.arange(len(marks)) % 4]
    return req


def complete_echo_reply(reply: np.ndarray, resp_size: int) -> int:
    """CompleteEchoReply, echo_client.cc:34-66: 0 when the reply has the agreed
    size and carries the pattern; otherwise 1 + the number of bytes that differ
    (the reference logs each of them)."""
    reply = np.asarray(reply, dtype=np.uint8).reshape(-1)
    if reply.size != resp_size:
        return 1
    bad = int(np.count_nonzero(reply != create_echo_request(resp_size)))
    return 0 if bad == 0 else 1 + bad


def create_vec_add_request(size: int) -> np.ndarray:
    """CreateEchoRequest, vec_add_client.cc:11-19."""
    return MAGIC_STRING[np.arange(size) % 4].copy()


def complete_vec_add_reply(reply: np.ndarray, resp_size: int) -> int:
    """CompleteEchoReply, vec_add_client.cc:21-33: every byte MAGIC[i % 4] + 1."""
    reply = np.asarray(reply, dtype=np.uint8).reshape(-1)
    if reply.size != resp_size:
        return 1
    want = (MAGIC_STRING[np.arange(resp_size) % 4].astype(np.uint16) + 1).astype(np.uint8)
    return 0 if np.array_equal(reply, want) else 1


def client_workload(kind: str, n_req: int, req_size: int, resp_size: Optional[int] = None, mtu: int = 1400,
                    slot_size: int = 2048, profile: int = synth.HDR_REF64, order: str = "shuffle_all",
                    seed: int = 77, flags: int = 0, n_slots: Optional[int] = None) -> synth.Workload:
    """``n_req`` requests of the ``kind`` client ("echo" or "vec_add") in a ring.

    echo: responses are written into the request's own buffers (the
    reference's zero-copy echo), so ``resp_size`` must equal ``req_size``.
    vec_add: responses go to a TX ring of their own; the expected response
    payload (request + 1) is what ``Workload.resp_payload`` holds."""
    resp_size = req_size if resp_size is None else resp_size
    rng = np.random.default_rng(seed)
    frames = synth.num_frames(req_size, mtu) * n_req
    if kind == "echo":
        assert resp_size == req_size, "the echo server answers in place"
        pay = [create_echo_request(req_size) for _ in range(n_req)]
        out, in_place = pay, True
    elif kind == "vec_add":
        pay = [create_vec_add_request(req_size) for _ in range(n_req)]
        full = (create_vec_add_request(max(req_size, resp_size)).astype(np.uint16) + 1).astype(np.uint8)
        out, in_place = [full[:resp_size].copy() for _ in range(n_req)], False
    else:
        raise ValueError(kind)
    return synth._assemble(kind, 0, seed, rng, profile, slot_size, n_slots or max(frames, 1), mtu, pay, order, 0,
                           [], out, [], flags, in_place, f"{kind} client, {n_req} x {req_size} B")


def verify_responses(w: synth.Workload, tx_ring: np.ndarray, kind: str) -> int:
    """Put every response back together from the TX ring's frames (in frame
    order, as the client's receive path does) and run the client's check on
    it.  Returns the number of responses that fail."""
    hl = synth.hdr_len(w.profile)
    tx = np.asarray(tx_ring, dtype=np.uint8).reshape(w.tx_n_slots, w.slot_size)
    check = complete_echo_reply if kind == "echo" else complete_vec_add_reply
    failed = 0
    for r in range(w.n_req):
        size = int(w.resp_sizes[r])
        parts = []
        for i, ln in enumerate(synth.frame_lens(size, w.mtu)):
            slot = int(w.tx_slot[int(w.resp_first[r]) + i])
            parts.append(tx[slot, hl:hl + int(ln)])
        reply = np.concatenate(parts) if parts else np.zeros(0, np.uint8)
        if check(reply, size) != 0:
            failed += 1
    return failed
