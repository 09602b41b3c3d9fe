"""Seeded synthetic packet rings for the five benchmark workloads.

A ring is ``n_slots`` fixed-size slots.  A slot holds one received frame: a
42-byte Ethernet/IPv4/UDP header, the RPC header of the chosen profile and the
payload; bytes past the payload are zero.  The NIC fills slots in arrival
order, so ``arrivals[k] = (head + k) % n_slots``.

Alongside the ring the generator emits what the receive thread of the
reference would have built from those arrivals (``P2pRpcRr`` fragment tables,
src/p2p_rpc_rr_ng.h:96-105, handed over in completion order,
src/p2p_rpc_rr_pool_ng.h:149-155) in compact CSR form:

``frag_slot[f]``   ring slot of fragment f (requests concatenated in batch
                   order, fragments in seq order inside a request)
``frag_len[f]``    payload bytes of fragment f
``req_first[r]``   first fragment of request r (n_req + 1 entries)

and the response side: per-request response bytes, the TX slots the response
frames go to and the RX slot each response frame takes its header from.

Only numpy is used; nothing here touches the GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

HDR_BL58 = 0
HDR_REF64 = 1

F_IPV4_CSUM = 1 << 0
F_UDP_CSUM_PSEUDO = 1 << 1
F_UDP_CSUM_FULL = 1 << 2
F_REF_QUIRKS = 1 << 3

L4_END = 42


def hdr_len(profile: int) -> int:
    return 64 if profile == HDR_REF64 else 58


def num_frames(size: int, mtu: int) -> int:
    """ceil(size / mtu): src/transport/dpdk_transport_ng.h:332."""
    return (int(size) + mtu - 1) // mtu


def frame_lens(size: int, mtu: int) -> np.ndarray:
    """Frame i carries min(remaining, mtu): src/transport/dpdk_rx_tx.h:137-139."""
    n = num_frames(size, mtu)
    lens = np.full(n, mtu, dtype=np.uint32)
    if n:
        lens[-1] = size - (n - 1) * mtu
    return lens


@dataclass
class Workload:
    name: str
    cfg: int
    seed: int
    profile: int
    slot_size: int
    n_slots: int
    mtu: int
    ring: np.ndarray  # uint8 [n_slots * slot_size]
    arrivals: np.ndarray  # uint32 [n_frags], slots in arrival order
    frag_slot: np.ndarray  # uint32 [n_frags]
    frag_len: np.ndarray  # uint32 [n_frags]
    req_first: np.ndarray  # uint32 [n_req + 1]
    req_ids: np.ndarray  # uint64 [n_req] in batch order
    req_sizes: np.ndarray  # uint64 [n_req] in batch order
    req_payload: np.ndarray  # uint8, requests concatenated in batch order
    in_tensor_sizes: List[int]  # tensor-major split of one request ([] = packed)
    # response side
    resp_sizes: np.ndarray  # uint64 [n_req]
    resp_payload: np.ndarray  # uint8, responses concatenated in batch order
    out_tensor_sizes: List[int]
    resp_first: np.ndarray  # uint32 [n_req + 1]
    tx_slot: np.ndarray  # uint32 [n_resp_frames]
    hdr_src_slot: np.ndarray  # uint32 [n_resp_frames], slots of the RX ring
    tx_n_slots: int
    tx_in_place: bool  # responses are written into the RX ring itself
    tx_ring_init: Optional[np.ndarray]  # uint8 initial TX ring bytes (None when in place)
    flags: int
    note: str = ""
    extra: dict = field(default_factory=dict)

    @property
    def n_req(self) -> int:
        return len(self.req_sizes)

    @property
    def n_frags(self) -> int:
        return len(self.frag_slot)

    @property
    def n_resp_frames(self) -> int:
        return len(self.tx_slot)

    def gather_bytes(self) -> int:
        """Algorithmic bytes of one gather pass: payload read + tensor write +
        16-byte RPC header read per frame."""
        return 2 * int(self.frag_len.sum(dtype=np.uint64)) + 16 * self.n_frags

    def scatter_bytes(self) -> int:
        """Algorithmic bytes of one scatter pass: output read + payload write +
        header read and write per response frame."""
        h = hdr_len(self.profile)
        return 2 * int(self.resp_sizes.sum(dtype=np.uint64)) + 2 * h * self.n_resp_frames


# --------------------------------------------------------------------------
# header construction
# --------------------------------------------------------------------------

def _ipv4_hdr_csum_rows(ip: np.ndarray) -> np.ndarray:
    """RFC 1071 over rows of 20-byte IPv4 headers (check field taken as 0)."""
    w = ip.astype(np.uint32)
    words = (w[:, 0::2] << 8) | w[:, 1::2]
    words[:, 5] = 0
    s = words.sum(axis=1)
    s = (s & 0xFFFF) + (s >> 16)
    s = (s & 0xFFFF) + (s >> 16)
    return (~s) & 0xFFFF


def build_headers(rng: np.random.Generator, profile: int, req_of_frag: np.ndarray,
                  frag_idx: np.ndarray, frags_of_req: np.ndarray, frag_len: np.ndarray,
                  req_ids: np.ndarray) -> np.ndarray:
    """One header per frame.  Every request has its own client MAC / IP / port;
    the server side is fixed.  Incoming frames carry a finished IPv4 checksum
    and an arbitrary UDP checksum word, as frames off a wire would."""
    n = len(req_of_frag)
    n_req = len(req_ids)
    hl = hdr_len(profile)
    h = np.zeros((n, hl), dtype=np.uint8)
    srv_mac = np.array([0xB8, 0xCE, 0xF6, 0xCC, 0x6A, 0x52], dtype=np.uint8)
    cli_mac = rng.integers(0, 256, size=(n_req, 6), dtype=np.uint8)
    cli_mac[:, 0] = (cli_mac[:, 0] & 0xFE) | 0x02  # locally administered unicast
    cli_ip = np.empty((n_req, 4), dtype=np.uint8)
    cli_ip[:, 0] = 10
    cli_ip[:, 1:] = rng.integers(1, 255, size=(n_req, 3), dtype=np.uint8)
    srv_ip = np.array([192, 168, 25, 1], dtype=np.uint8)
    cli_port = rng.integers(1024, 65536, size=n_req, dtype=np.uint32)
    srv_port = 50051
    ip_id = rng.integers(0, 65536, size=n, dtype=np.uint32)
    udp_ck = rng.integers(1, 65536, size=n, dtype=np.uint32)

    r = req_of_frag
    h[:, 0:6] = srv_mac
    h[:, 6:12] = cli_mac[r]
    h[:, 12] = 0x08
    h[:, 13] = 0x00
    h[:, 14] = 0x45
    h[:, 15] = 0x00
    tail = hl - L4_END
    tot = (28 + tail + frag_len).astype(np.uint32)
    h[:, 16] = tot >> 8
    h[:, 17] = tot & 0xFF
    h[:, 18] = ip_id >> 8
    h[:, 19] = ip_id & 0xFF
    h[:, 20] = 0x40  # don't fragment
    h[:, 21] = 0
    h[:, 22] = 64
    h[:, 23] = 17
    h[:, 26:30] = cli_ip[r]
    h[:, 30:34] = srv_ip
    ck = _ipv4_hdr_csum_rows(h[:, 14:34])
    h[:, 24] = ck >> 8
    h[:, 25] = ck & 0xFF
    h[:, 34] = cli_port[r] >> 8
    h[:, 35] = cli_port[r] & 0xFF
    h[:, 36] = srv_port >> 8
    h[:, 37] = srv_port & 0xFF
    ul = (8 + tail + frag_len).astype(np.uint32)
    h[:, 38] = ul >> 8
    h[:, 39] = ul & 0xFF
    h[:, 40] = udp_ck >> 8
    h[:, 41] = udp_ck & 0xFF
    h[:, 42:50] = req_ids[r].astype("<u8").view(np.uint8).reshape(-1, 8)
    if profile == HDR_BL58:
        h[:, 50:52] = frag_idx.astype("<u2").view(np.uint8).reshape(-1, 2)
        h[:, 52:54] = frags_of_req[r].astype("<u2").view(np.uint8).reshape(-1, 2)
        h[:, 54:58] = frag_len.astype("<u4").view(np.uint8).reshape(-1, 4)
    else:
        sp = rng.integers(0, 2 ** 63, size=n, dtype=np.int64)
        h[:, 50:58] = sp.astype("<i8").view(np.uint8).reshape(-1, 8)
        h[:, 58:60] = frag_idx.astype("<u2").view(np.uint8).reshape(-1, 2)
    return h


# --------------------------------------------------------------------------
# ring assembly
# --------------------------------------------------------------------------

def _assemble(name: str, cfg: int, seed: int, rng: np.random.Generator, profile: int,
              slot_size: int, n_slots: int, mtu: int, payloads: List[np.ndarray],
              order: str, head: int, in_tensor_sizes: List[int], resp: List[np.ndarray],
              out_tensor_sizes: List[int], flags: int, in_place: bool, note: str,
              tx_n_slots: Optional[int] = None) -> Workload:
    """payloads[i] / resp[i] are request i's bytes in *generation* order; the
    batch order is the order in which requests complete."""
    n_req = len(payloads)
    hl = hdr_len(profile)
    assert hl + mtu <= slot_size
    sizes = np.array([len(p) for p in payloads], dtype=np.uint64)
    nfr = np.array([num_frames(int(s), mtu) for s in sizes], dtype=np.uint32)
    assert nfr.max(initial=0) <= 1023, "a reference run table describes at most 1023 runs"
    first = np.zeros(n_req + 1, dtype=np.int64)
    np.cumsum(nfr, out=first[1:])
    n_frags = int(first[-1])
    assert n_frags <= n_slots
    req_of_frag = np.repeat(np.arange(n_req, dtype=np.int64), nfr)
    frag_idx = (np.arange(n_frags, dtype=np.int64) - first[req_of_frag]).astype(np.uint32)
    flen = np.concatenate([frame_lens(int(s), mtu) for s in sizes]) if n_req else np.zeros(0, np.uint32)

    # arrival position of every frame (generation-order frame index -> position)
    if order == "in_order":
        pos = np.arange(n_frags, dtype=np.int64)
    elif order == "perm_within_request":
        pos = np.empty(n_frags, dtype=np.int64)
        for r in range(n_req):
            a, b = int(first[r]), int(first[r + 1])
            pos[a:b] = a + rng.permutation(b - a)
    elif order == "interleave_keep_order":
        p = rng.permutation(n_frags)
        pos = np.empty(n_frags, dtype=np.int64)
        for r in range(n_req):
            a, b = int(first[r]), int(first[r + 1])
            pos[a:b] = np.sort(p[a:b])
    elif order == "shuffle_all":
        pos = rng.permutation(n_frags).astype(np.int64)
    else:
        raise ValueError(order)
    slot_of_frag = ((head + pos) % n_slots).astype(np.uint32)
    arrivals = ((head + np.arange(n_frags, dtype=np.int64)) % n_slots).astype(np.uint32)

    req_ids_gen = (np.uint64(0x1000_0000_0000) * np.uint64(cfg + 1)
                   + rng.permutation(n_req).astype(np.uint64) + np.uint64(1))
    headers = build_headers(rng, profile, req_of_frag, frag_idx, nfr, flen, req_ids_gen)

    ring = np.zeros((n_slots, slot_size), dtype=np.uint8)
    ring[slot_of_frag, :hl] = headers
    for r in range(n_req):
        a, b = int(first[r]), int(first[r + 1])
        if a == b:
            continue
        padded = np.zeros((b - a) * mtu, dtype=np.uint8)
        padded[: len(payloads[r])] = payloads[r]
        ring[slot_of_frag[a:b], hl:hl + mtu] = padded.reshape(b - a, mtu)

    # completion order: a request completes when its last frame arrives
    done_pos = np.array([pos[int(first[r]):int(first[r + 1])].max(initial=-1) for r in range(n_req)])
    batch = np.argsort(done_pos, kind="stable")

    b_first = np.zeros(n_req + 1, dtype=np.uint32)
    np.cumsum(nfr[batch], out=b_first[1:])
    gen_idx = np.concatenate([np.arange(first[r], first[r + 1]) for r in batch]) if n_req else np.zeros(0, np.int64)
    frag_slot = slot_of_frag[gen_idx]
    frag_len = flen[gen_idx]
    req_payload = np.concatenate([payloads[r] for r in batch]) if n_req else np.zeros(0, np.uint8)

    # responses
    rsz = np.array([len(resp[r]) for r in batch], dtype=np.uint64)
    rnf = np.array([num_frames(int(s), mtu) for s in rsz], dtype=np.uint32)
    r_first = np.zeros(n_req + 1, dtype=np.uint32)
    np.cumsum(rnf, out=r_first[1:])
    n_rf = int(r_first[-1])
    resp_payload = np.concatenate([resp[r] for r in batch]) if n_req else np.zeros(0, np.uint8)
    if in_place:
        # echo: response frame i reuses the slot of request frame i
        assert np.array_equal(rnf, nfr[batch])
        tx_slot = frag_slot.copy()
        hdr_src = frag_slot.copy()
        tx_slots = n_slots
        tx_init = None
    else:
        tx_slots = tx_n_slots if tx_n_slots is not None else max(n_rf, 1)
        assert n_rf <= tx_slots
        tx_slot = rng.permutation(tx_slots)[:n_rf].astype(np.uint32)
        # header of response frame i comes from request frame (i mod request frames)
        hdr_src = np.empty(n_rf, dtype=np.uint32)
        for k in range(n_req):
            a, b = int(r_first[k]), int(r_first[k + 1])
            fa, fb = int(b_first[k]), int(b_first[k + 1])
            hdr_src[a:b] = frag_slot[fa + (np.arange(b - a) % max(fb - fa, 1))]
        tx_init = rng.integers(0, 256, size=tx_slots * slot_size, dtype=np.uint8)

    return Workload(
        name=name, cfg=cfg, seed=seed, profile=profile, slot_size=slot_size, n_slots=n_slots,
        mtu=mtu, ring=ring.reshape(-1), arrivals=arrivals, frag_slot=frag_slot,
        frag_len=frag_len, req_first=b_first, req_ids=req_ids_gen[batch],
        req_sizes=sizes[batch], req_payload=req_payload, in_tensor_sizes=in_tensor_sizes,
        resp_sizes=rsz, resp_payload=resp_payload, out_tensor_sizes=out_tensor_sizes,
        resp_first=r_first, tx_slot=tx_slot, hdr_src_slot=hdr_src, tx_n_slots=tx_slots,
        tx_in_place=in_place, tx_ring_init=tx_init, flags=flags, note=note)


def _bytes(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1)


SEED_BASE = 0x5EED0000


def make_workload(cfg: int, n_req: Optional[int] = None, seed: Optional[int] = None,
                  profile: int = HDR_BL58) -> Workload:
    """Workloads 1..5 at their nominal size (``n_req=None``) or scaled down to
    ``n_req`` requests with everything else unchanged."""
    seed = SEED_BASE + cfg if seed is None else seed
    rng = np.random.default_rng(seed)
    if cfg == 1:
        n = 32 if n_req is None else n_req
        pay = [_bytes(rng.random(28 * 28, dtype=np.float32)) for _ in range(n)]
        out = [_bytes(rng.standard_normal(10).astype(np.float32)) for _ in range(n)]
        return _assemble("lenet", 1, seed, rng, profile, 2048, 3 * n, 1400, pay, "in_order", 0,
                         [], out, [], F_UDP_CSUM_PSEUDO, False,
                         "28x28 fp32 U[0,1) -> 10 fp32; frames in order")
    if cfg == 2:
        n = 16 if n_req is None else n_req
        pay = [_bytes(rng.standard_normal(3 * 224 * 224, dtype=np.float32)) for _ in range(n)]
        out = [_bytes(rng.standard_normal(1000, dtype=np.float32)) for _ in range(n)]
        return _assemble("resnet50", 2, seed, rng, profile, 2048, 431 * n, 1400, pay,
                         "perm_within_request", 0, [], out, [], F_IPV4_CSUM | F_UDP_CSUM_PSEUDO,
                         False, "3x224x224 fp32 N(0,1) -> 1000 fp32; permuted inside a request")
    if cfg == 3:
        n = 256 if n_req is None else n_req
        pay = []
        for _ in range(n):
            ids = rng.integers(0, 30522, size=128, dtype=np.int64)
            ln = int(rng.integers(16, 129))
            mask = np.zeros(128, dtype=np.int64)
            mask[:ln] = 1
            pay.append(np.concatenate([_bytes(ids), _bytes(mask)]))
        out = [_bytes(rng.standard_normal(768, dtype=np.float32)) for _ in range(n)]
        slots = max(1024, 1 << int(np.ceil(np.log2(max(2 * n, 2))))) if n_req is None else max(4 * n, 8)
        head = int(rng.integers(0, slots))
        return _assemble("bert", 3, seed, rng, profile, 2048, slots, 1400, pay,
                         "interleave_keep_order", head, [1024, 1024], out, [3072],
                         F_UDP_CSUM_PSEUDO, False,
                         "128 int64 ids + 128 int64 mask -> 768 fp32; requests interleaved")
    if cfg == 4:
        n = 4096 if n_req is None else n_req
        sizes = np.rint(np.exp(rng.uniform(np.log(64.0), np.log(65536.0), size=n))).astype(np.int64)
        pay = [rng.integers(0, 256, size=int(s), dtype=np.uint8) for s in sizes]
        slots = 65536 if n_req is None else max(64, 1 << int(np.ceil(np.log2(max(int(np.sum((sizes + 1399) // 1400)), 2)) + 1)))
        head = int(rng.integers(0, slots))
        return _assemble("mixed", 4, seed, rng, profile, 2048, slots, 1400, pay, "shuffle_all",
                         head, [], pay, [], F_UDP_CSUM_PSEUDO, True,
                         "log-uniform 64 B..64 KiB random bytes, echoed in place")
    if cfg == 5:
        n = 64 if n_req is None else n_req
        pay = [_bytes(rng.standard_normal(3 * 512 * 512, dtype=np.float32).astype(np.float16))
               for _ in range(n)]
        out = [_bytes(rng.integers(0, 21, size=512 * 512, dtype=np.int32)) for _ in range(n)]
        return _assemble("jumbo", 5, seed, rng, profile, 9216, 179 * n, 8800, pay, "shuffle_all", 0,
                         [], out, [], F_IPV4_CSUM | F_UDP_CSUM_FULL, False,
                         "3x512x512 fp16 N(0,1) -> 512x512 int32; jumbo frames, full UDP checksum")
    raise ValueError(f"unknown workload {cfg}")


def make_custom(sizes, resp_sizes, mtu=1400, slot_size=2048, n_slots=None, order="shuffle_all",
                seed=1234, profile=HDR_BL58, in_tensor_sizes=(), out_tensor_sizes=(), flags=0,
                in_place=False, head=0, tx_n_slots=None) -> Workload:
    """Arbitrary request / response sizes with random bytes: edge-case rings."""
    rng = np.random.default_rng(seed)
    pay = [rng.integers(0, 256, size=int(s), dtype=np.uint8) for s in sizes]
    out = pay if in_place else [rng.integers(0, 256, size=int(s), dtype=np.uint8) for s in resp_sizes]
    nfr = sum(num_frames(int(s), mtu) for s in sizes)
    if n_slots is None:
        n_slots = max(nfr, 1)
    return _assemble("custom", 0, seed, rng, profile, slot_size, n_slots, mtu, pay, order, head,
                     list(in_tensor_sizes), out, list(out_tensor_sizes), flags, in_place, "custom",
                     tx_n_slots=tx_n_slots)
