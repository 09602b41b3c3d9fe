"""Pins of the CPU oracle: every function of oracle/sg_oracle.c is held against
something it cannot have inherited its own mistakes from -- the compiled
reference headers (oracle/_ref, built where the reference tree is present), a
textbook vector, an invariant of the standard, or a brute-force restatement in
another arithmetic domain (big-endian words, pure-Python loops)."""
import ctypes as C
import hashlib
import json
import os

import numpy as np
import pytest

import oracle
from splitrpc_amd import synth

L = oracle.lib()
REF = oracle.ref()
needs_ref = pytest.mark.skipif(REF is None, reason="reference probe not built (no reference tree here)")


def p(a):
    return a.ctypes.data_as(C.c_void_p)


def rand_hdr(rng, n=64):
    h = rng.integers(0, 256, n, dtype=np.uint8)
    h[14] = 0x45
    h[23] = 17
    return h


def be_sum(b):
    """One's-complement sum of big-endian 16-bit words, folded."""
    b = bytes(b)
    if len(b) & 1:
        b += b"\0"
    s = sum((b[i] << 8) | b[i + 1] for i in range(0, len(b), 2))
    while s >> 16:
        s = (s & 0xFFFF) + (s >> 16)
    return s


def bswap16(v):
    return ((v & 0xFF) << 8) | (v >> 8)


# ---------------------------------------------------------------- layouts

@needs_ref
def test_table_and_wire_layouts_match_compiled_reference():
    got = [REF.ref_layout(i) for i in range(27)]
    assert got[0] == C.sizeof(oracle.HBufs) == 8194
    assert got[1] == C.sizeof(oracle.Bufs) == 16386
    assert got[2] == C.sizeof(oracle.SkBuf) == 24576
    assert got[3] == 16 and got[4] == 128
    assert got[5:9] == [14, 20, 8, 42]
    assert got[9] == oracle.MAX_BI_SIZE == 1024
    assert got[10] == oracle.HBufs.num_items.offset
    assert got[11] == oracle.Bufs.item_size.offset
    assert got[12] == oracle.Bufs.num_items.offset
    assert got[13] == oracle.SkBuf.o_buf.offset
    assert got[14] == oracle.SkBuf.len.offset
    assert got[15] == oracle.SkBuf.num_items.offset
    # ipv4 / udp field offsets the restatement hard-codes (relative to the L3 / L4 header)
    assert got[20:24] == [2, 10, 12, 16] and got[24:27] == [4, 6, 9]


def test_abi_tables_match_oracle_tables():
    from splitrpc_amd import capi
    assert C.sizeof(capi.SkBuf) == C.sizeof(oracle.SkBuf) == 24576
    assert C.sizeof(capi.HBufs) == C.sizeof(oracle.HBufs) == 8194


# ---------------------------------------------------------------- pseudo sum

@needs_ref
def test_pseudo_csum_matches_compiled_reference():
    """eth_common.h:92-130 sums 16 bytes of which it writes 12; with the stack
    below it painted zero the compiled reference gives the oracle's quirk value."""
    rng = np.random.default_rng(11)
    for _ in range(3000):
        ip = rng.integers(0, 256, 20, dtype=np.uint8)
        ip[0] = 0x45
        assert REF.ref_ipv4_pseudo_csum(p(ip), 0) == L.sgo_ipv4_pseudo_csum(p(ip), 1)


@needs_ref
def test_pseudo_csum_reference_reads_unwritten_bytes():
    """The four bytes the reference never writes take part in its sum: painting
    the stack with another value moves the result by exactly those two words."""
    ip = np.array([0x45, 0, 0x05, 0xB4, 0, 0, 0x40, 0, 64, 17, 0, 0, 10, 1, 2, 3, 192, 168, 25, 1], np.uint8)
    clean = REF.ref_ipv4_pseudo_csum(p(ip), 0)
    dirty = REF.ref_ipv4_pseudo_csum(p(ip), 0x21)
    s = clean + 0x2121 + 0x2121
    s = (s & 0xFFFF) + (s >> 16)
    s = (s & 0xFFFF) + (s >> 16)
    assert dirty == s and dirty != clean


@needs_ref
def test_version_nibble_is_what_the_quirk_subtracts():
    ihl, ver = C.c_int(), C.c_int()
    ip = np.zeros(20, np.uint8)
    ip[0] = 0x45
    REF.ref_ip_nibbles(p(ip), C.byref(ihl), C.byref(ver))
    assert (ihl.value, ver.value) == (5, 4)  # so version * 4 == 16, not the 20 header bytes


def test_pseudo_csum_by_hand():
    # 10.1.2.3 -> 192.168.25.1, UDP, tot_len 1444: big-endian words by hand
    ip = np.array([0x45, 0, 0x05, 0xA4, 0, 0, 0x40, 0, 64, 17, 0, 0, 10, 1, 2, 3, 192, 168, 25, 1], np.uint8)
    words = [0x0A01, 0x0203, 0xC0A8, 0x1901, 0x0011]
    for quirk, sub in ((0, 20), (1, 16)):
        s = sum(words) + (1444 - sub)
        while s >> 16:
            s = (s & 0xFFFF) + (s >> 16)
        # the function sums little-endian words and returns the native value
        assert L.sgo_ipv4_pseudo_csum(p(ip), quirk) == bswap16(s)


def test_pseudo_csum_against_big_endian_restatement():
    rng = np.random.default_rng(5)
    for _ in range(500):
        ip = rng.integers(0, 256, 20, dtype=np.uint8)
        ip[0] = 0x45
        tot = int(rng.integers(28, 65000))
        ip[2], ip[3] = tot >> 8, tot & 0xFF
        ln = tot - 20
        psd = bytes(ip[12:20]) + bytes([0, ip[9], ln >> 8, ln & 0xFF])
        assert L.sgo_ipv4_pseudo_csum(p(ip), 0) == bswap16(be_sum(psd))


# ---------------------------------------------------------------- header rewrite

def test_swap_is_an_involution_and_leaves_the_rest_alone():
    rng = np.random.default_rng(3)
    for _ in range(200):
        h0 = rand_hdr(rng)
        h = h0.copy()
        L.sgo_swap_eth_hdr(p(h))
        assert bytes(h[0:6]) == bytes(h0[6:12]) and bytes(h[6:12]) == bytes(h0[0:6])
        assert bytes(h[26:30]) == bytes(h0[30:34]) and bytes(h[30:34]) == bytes(h0[26:30])
        assert bytes(h[34:36]) == bytes(h0[36:38]) and bytes(h[36:38]) == bytes(h0[34:36])
        assert h[24] == h[25] == h[40] == h[41] == 0
        untouched = list(range(12, 24)) + [38, 39] + list(range(42, 64))
        assert np.array_equal(h[untouched], h0[untouched])
        L.sgo_swap_eth_hdr(p(h))
        keep = [i for i in range(64) if i not in (24, 25, 40, 41)]
        assert np.array_equal(h[keep], h0[keep])


def test_swap_hand_vector():
    h = np.arange(64, dtype=np.uint8)
    L.sgo_swap_eth_hdr(p(h))
    want = list(range(6, 12)) + list(range(0, 6)) + list(range(12, 24)) + [0, 0] + \
        list(range(30, 34)) + list(range(26, 30)) + [36, 37, 34, 35, 38, 39, 0, 0] + list(range(42, 64))
    assert h.tolist() == want


def test_lengths_closed_form():
    for L_ in (0, 16, 22, 1416, 1422, 8816, 65000):
        h = np.zeros(64, np.uint8)
        L.sgo_add_ip_udp_len(p(h), L_)
        assert (int(h[16]) << 8 | int(h[17])) == 28 + L_
        assert (int(h[38]) << 8 | int(h[39])) == 8 + L_


def test_sockperf_and_conn_info():
    rng = np.random.default_rng(9)
    h = rand_hdr(rng)
    h0 = h.copy()
    L.sgo_set_sockperf_header(p(h))
    assert np.array_equal(h[50:54], np.zeros(4, np.uint8)) and np.array_equal(h[54:58], h0[54:58])
    assert np.array_equal(np.delete(h, range(50, 54)), np.delete(h0, range(50, 54)))
    for prof, hl in ((synth.HDR_BL58, 58), (synth.HDR_REF64, 64)):
        tmpl, recv = rand_hdr(rng), rand_hdr(rng)
        t0 = tmpl.copy()
        L.sgo_set_conn_info(p(tmpl), p(recv), prof)
        assert np.array_equal(tmpl[42:hl], recv[42:hl])        # RPC tail of the first packet
        assert np.array_equal(tmpl[36:38], recv[34:36])        # dst port <- src port
        assert np.array_equal(tmpl[30:34], recv[26:30])        # dst ip <- src ip
        assert np.array_equal(tmpl[0:6], recv[6:12])           # dst mac <- src mac
        same = list(range(6, 30)) + [34, 35] + list(range(38, 42)) + list(range(hl, 64))
        assert np.array_equal(tmpl[same], t0[same])


@pytest.mark.parametrize("prof,hl", [(synth.HDR_BL58, 58), (synth.HDR_REF64, 64)])
def test_template_header_equals_swapped_header_on_one_connection(prof, hl):
    """rr_set_hdr (template copy) and rr_swap_hdr (in-place swap) are two ways
    to the same response header: when the server's template carries the
    identity the request was sent to, they must agree byte for byte.  A wrong
    offset in either path, or in set_conn_info, breaks the equality."""
    rng = np.random.default_rng(31)
    for it in range(40):
        cm, sm = rng.integers(0, 256, 6, dtype=np.uint8), rng.integers(0, 256, 6, dtype=np.uint8)
        cip, sip = int(rng.integers(0, 2 ** 32)), int(rng.integers(0, 2 ** 32))
        cp, sp = int(rng.integers(0, 65536)), int(rng.integers(0, 65536))
        req = np.zeros(64, np.uint8)
        L.sgo_gen_hdr_template(p(req), p(cm), p(sm), cip, sip, cp, sp)       # client -> server
        req[42:64] = rng.integers(0, 256, 22, dtype=np.uint8)
        tmpl = np.zeros(64, np.uint8)
        other = rng.integers(0, 256, 6, dtype=np.uint8)
        L.sgo_gen_hdr_template(p(tmpl), p(sm), p(other), sip, 0x01020304, sp, 9)  # server -> nobody yet
        L.sgo_set_conn_info(p(tmpl), p(req), prof)
        token = int(req[42:50].view(np.uint64)[0])
        for flags in (0, 1, 2, 3, 10):
            for idx, n, plen in ((0, 1, 1), (3, 7, 1400), (1022, 1023, 777)):
                a, b = req.copy(), np.zeros(64, np.uint8)
                L.sgo_rewrite_resp_hdr(p(a), prof, flags, idx, n, plen)
                L.sgo_template_resp_hdr(p(b), p(tmpl), prof, flags, token, idx, n, plen)
                assert np.array_equal(a[:hl], b[:hl]), (it, flags, idx, np.flatnonzero(a[:hl] != b[:hl]))
        # and the token argument really lands in bytes 42..49
        b = np.zeros(64, np.uint8)
        L.sgo_template_resp_hdr(p(b), p(tmpl), prof, 0, 0x1122334455667788, 0, 1, 5)
        assert bytes(b[42:50]) == (0x1122334455667788).to_bytes(8, "little")


@needs_ref
def test_header_template_matches_compiled_reference():
    rng = np.random.default_rng(2)
    for _ in range(50):
        sm, dm = rng.integers(0, 256, 6, dtype=np.uint8), rng.integers(0, 256, 6, dtype=np.uint8)
        sip, dip = int(rng.integers(0, 2 ** 32)), int(rng.integers(0, 2 ** 32))
        sp, dp = int(rng.integers(0, 65536)), int(rng.integers(0, 65536))
        a, b = np.zeros(42, np.uint8), np.zeros(42, np.uint8)
        REF.ref_gen_hdr_template(p(a), p(sm), p(dm), sip, dip, sp, dp)
        L.sgo_gen_hdr_template(p(b), p(sm), p(dm), sip, dip, sp, dp)
        assert np.array_equal(a, b)


# ---------------------------------------------------------------- finished checksums (RFC 1071 / 768)

def test_ipv4_header_checksum_textbook_vector():
    hdr = bytes.fromhex("450000730000400040110000c0a80001c0a800c7")
    ip = np.frombuffer(hdr, np.uint8).copy()
    ck = L.sgo_ipv4_hdr_csum(p(ip))
    ip[10:12] = np.frombuffer(int(ck).to_bytes(2, "little"), np.uint8)  # stored natively
    assert bytes(ip[10:12]).hex() == "b861"
    assert be_sum(ip) == 0xFFFF


def test_ipv4_header_checksum_verifies_to_ffff_and_ignores_old_field():
    rng = np.random.default_rng(4)
    for _ in range(300):
        ip = rng.integers(0, 256, 20, dtype=np.uint8)
        ip[0] = 0x45
        ck = L.sgo_ipv4_hdr_csum(p(ip))
        ip2 = ip.copy()
        ip2[10:12] = 0
        assert L.sgo_ipv4_hdr_csum(p(ip2)) == ck
        ip2[10:12] = np.frombuffer(int(ck).to_bytes(2, "little"), np.uint8)
        assert be_sum(ip2) == 0xFFFF


def _udp_packet(rng, n_payload, profile_tail=16):
    ip = rng.integers(0, 256, 20, dtype=np.uint8)
    ip[0] = 0x45
    ip[9] = 17
    ulen = 8 + profile_tail + n_payload
    udp = rng.integers(0, 256, ulen, dtype=np.uint8)
    udp[4], udp[5] = ulen >> 8, ulen & 0xFF
    pkt = np.concatenate([ip, udp])
    return pkt, ulen


def test_udp_checksum_against_scalar_restatement_and_ffff():
    rng = np.random.default_rng(6)
    for n in (0, 1, 2, 3, 17, 112, 1399, 1400, 8799, 8800):
        pkt, ulen = _udp_packet(rng, n)
        ck = L.sgo_udp_full_csum(p(pkt), p(pkt[20:]))
        # RFC 768: pseudo header + UDP header with zero check + data, padded
        seg = bytearray(pkt[20:20 + ulen])
        seg[6:8] = b"\0\0"
        psd = bytes(pkt[12:20]) + bytes([0, 17, ulen >> 8, ulen & 0xFF])
        want = (~be_sum(psd + bytes(seg) + (b"\0" if ulen & 1 else b""))) & 0xFFFF
        want = want or 0xFFFF
        assert ck == bswap16(want)
        # a receiver summing everything including the checksum sees 0xffff
        seg[6:8] = want.to_bytes(2, "big")
        assert be_sum(psd + bytes(seg) + (b"\0" if ulen & 1 else b"")) == 0xFFFF


def test_udp_checksum_zero_is_sent_as_ffff():
    rng = np.random.default_rng(8)
    pkt, ulen = _udp_packet(rng, 32)
    seg = bytearray(pkt[20:20 + ulen])
    seg[6:8] = b"\0\0"
    psd = bytes(pkt[12:20]) + bytes([0, 17, ulen >> 8, ulen & 0xFF])
    s = be_sum(psd + bytes(seg))
    # steer the last payload word so that the folded sum becomes 0xffff (checksum 0)
    last = (seg[-2] << 8) | seg[-1]
    rest = (s - last) if s >= last else (s - last + 0xFFFF)
    new_last = (0xFFFF - rest) & 0xFFFF
    pkt[20 + ulen - 2], pkt[20 + ulen - 1] = new_last >> 8, new_last & 0xFF
    assert L.sgo_udp_full_csum(p(pkt), p(pkt[20:])) == 0xFFFF


# ---------------------------------------------------------------- run descriptors

def _bufs(ptrs, sizes):
    b = oracle.Bufs()
    for i, (q, s) in enumerate(zip(ptrs, sizes)):
        b.burst_items[i] = q
        b.item_size[i] = s
    b.num_items = len(ptrs)
    return b


def test_gather_skbs_closed_form_and_merge_rule():
    rng = np.random.default_rng(12)
    for _ in range(200):
        n = int(rng.integers(1, 40))
        sizes = rng.integers(1, 2000, n).tolist()
        ptrs, cur = [], 1 << 20
        for i in range(n):
            if i and rng.random() < 0.4:
                cur = ptrs[-1] + sizes[i - 1]          # abuts the previous fragment
            else:
                cur = cur + int(rng.integers(3000, 9000))
            ptrs.append(cur)
        skb, b = oracle.SkBuf(), _bufs(ptrs, sizes)
        L.sgo_gather_skbs(C.byref(skb), C.byref(b), 7777)
        runs = [(skb.i_buf[k], skb.o_buf[k], skb.len[k]) for k in range(skb.num_items)]
        # expanding the runs gives back every fragment at the running sum of the sizes
        flat, off = [], 0
        for q, s in zip(ptrs, sizes):
            flat.append((q, 7777 + off, s))
            off += s
        k, used = 0, 0
        for q, o, s in flat:
            src, dst, ln = runs[k]
            assert (src + used, dst + used) == (q, o)
            used += s
            if used == ln:
                k, used = k + 1, 0
        assert k == len(runs)
        # a new run starts exactly where a fragment does not abut its predecessor
        breaks = 1 + sum(1 for i in range(1, n) if ptrs[i] != ptrs[i - 1] + sizes[i - 1])
        assert len(runs) == breaks
        # scatter is the mirror image
        skb2 = oracle.SkBuf()
        L.sgo_scatter_skbs(C.byref(skb2), C.byref(b), 7777)
        assert [(skb2.o_buf[k], skb2.i_buf[k], skb2.len[k]) for k in range(skb2.num_items)] == runs


def test_gather_skbs_emits_entry_zero_for_an_empty_table():
    """The reference writes entry 0 and returns num_items 1 even for an empty
    table (p2p_rpc_sg_engine.h:23-28,44): restated as is."""
    skb, b = oracle.SkBuf(), _bufs([123], [45])
    b.num_items = 0
    L.sgo_gather_skbs(C.byref(skb), C.byref(b), 1000)
    assert skb.num_items == 1 and (skb.i_buf[0], skb.o_buf[0], skb.len[0]) == (123, 1000, 45)


def test_sg_on_cpu_moves_the_runs():
    rng = np.random.default_rng(13)
    src = rng.integers(0, 256, 5000, dtype=np.uint8)
    dst = np.zeros(5000, np.uint8)
    skb = oracle.SkBuf()
    pieces = [(100, 0, 700), (2000, 700, 1), (3000, 701, 1400)]
    for k, (s, d, n) in enumerate(pieces):
        skb.i_buf[k], skb.o_buf[k], skb.len[k] = src.ctypes.data + s, dst.ctypes.data + d, n
    skb.num_items = len(pieces)
    L.sgo_sg_on_cpu(C.byref(skb))
    want = np.zeros(5000, np.uint8)
    for s, d, n in pieces:
        want[d:d + n] = src[s:s + n]
    assert np.array_equal(dst, want)


# ---------------------------------------------------------------- fragmenting rule, bump ring

def test_fragmenting_rule():
    for size, mtu in ((0, 1400), (1, 1400), (1399, 1400), (1400, 1400), (1401, 1400), (602112, 1400),
                      (1572864, 8800), (4000, 1400), (3136, 1400)):
        n = L.sgo_num_frames(size, mtu)
        assert n == -(-size // mtu)
        rem, lens = size, []
        for i in range(n):                       # the loop of dpdk_rx_tx.h:137-139
            cur = rem if rem <= mtu else mtu
            rem -= cur
            lens.append(cur)
        assert [L.sgo_frame_len(size, mtu, i) for i in range(n)] == lens
        assert sum(lens) == size and np.array_equal(synth.frame_lens(size, mtu), lens)


@needs_ref
def test_tring_matches_compiled_reference():
    rng = np.random.default_rng(14)
    for cap in (4096, 602112 * 7, 1000003):
        sizes = rng.integers(1, cap // 3, 200).astype(np.uint64)
        out = np.zeros(200, np.uint64)
        REF.ref_tring_replay(1 << 30, cap, p(sizes), 200, p(out))
        t = oracle.Tring()
        L.sgo_tring_init(C.byref(t), 1 << 30, cap)
        mine = [L.sgo_tring_get_next(C.byref(t), int(s)) for s in sizes]
        assert mine == out.tolist()


def test_tring_closed_form():
    t = oracle.Tring()
    L.sgo_tring_init(C.byref(t), 5000, 1000)
    sizes = [300, 300, 300, 300, 1, 999]
    want, off = [], 0
    for s in sizes:
        want.append(5000 + off)
        off = (off + s) % 1000
    assert [L.sgo_tring_get_next(C.byref(t), s) for s in sizes] == want


# ---------------------------------------------------------------- reassembly

def _py_reassemble(w, arrivals, len_nic=None, req_size=0):
    """Brute force: group slots by token in arrival order, index by the
    fragment's sequence number.  BL58: complete when num_frags fragments are in.
    REF64 (the reference's header: seq_num at byte 58, no count, no length):
    lengths come per slot as from the NIC and a request is complete when its
    bytes add up to the server-wide request size (src/p2p_rpc_rr_ng.h:107-110)."""
    ring = w.ring.reshape(w.n_slots, w.slot_size)
    live, done = {}, []
    for s in arrivals:
        h = ring[s]
        tok = int.from_bytes(bytes(h[42:50]), "little")
        if tok == 0:
            continue
        if w.profile == synth.HDR_REF64:
            idx = int.from_bytes(bytes(h[58:60]), "little")
            ln = int(len_nic[s])
        else:
            idx = int.from_bytes(bytes(h[50:52]), "little")
            nf = int.from_bytes(bytes(h[52:54]), "little")
            ln = int.from_bytes(bytes(h[54:58]), "little")
        d = live.setdefault(tok, {})
        d[idx] = (int(s), ln)
        ready = (sum(l for _, l in d.values()) == req_size) if w.profile == synth.HDR_REF64 else (len(d) == nf)
        if ready:
            done.append((tok, [d[i] for i in range(len(d))]))
            del live[tok]
    return done


@pytest.mark.parametrize("cfg,n", [(1, 8), (2, 2), (5, 2)])
def test_reassembly_by_request_size_against_brute_force(cfg, n):
    """The REF64 completion rule of the oracle, against the brute force above,
    in generated order and shuffled."""
    w = synth.make_workload(cfg, n, profile=synth.HDR_REF64)
    len_nic = np.zeros(w.n_slots, np.uint32)
    len_nic[w.frag_slot] = w.frag_len
    size = int(w.req_sizes[0])
    for arr in (w.arrivals, np.random.default_rng(cfg).permutation(w.arrivals)):
        fs, fl, rf, tok = oracle.reassemble(w, arrivals=arr, req_size=size, frag_len_nic=len_nic)
        want = _py_reassemble(w, arr, len_nic, size)
        assert len(want) == n
        assert tok.tolist() == [t for t, _ in want]
        assert fs.tolist() == [s for _, fr in want for s, _ in fr]
        assert fl.tolist() == [l for _, fr in want for _, l in fr]
        assert rf.tolist() == np.concatenate([[0], np.cumsum([len(fr) for _, fr in want])]).tolist()


@pytest.mark.parametrize("cfg,n", [(1, 8), (2, 2), (3, 40), (4, 60), (5, 2)])
def test_reassembly_against_brute_force(cfg, n):
    w = synth.make_workload(cfg, n)
    fs, fl, rf, tok = oracle.reassemble(w)
    want = _py_reassemble(w, w.arrivals)
    assert tok.tolist() == [t for t, _ in want]
    assert fs.tolist() == [s for _, fr in want for s, _ in fr]
    assert fl.tolist() == [l for _, fr in want for _, l in fr]
    assert rf.tolist() == np.concatenate([[0], np.cumsum([len(fr) for _, fr in want])]).tolist()
    # and the generator's own tables say the same
    assert np.array_equal(fs, w.frag_slot) and np.array_equal(rf, w.req_first)
    assert np.array_equal(tok, w.req_ids)


def test_reassembled_payload_does_not_depend_on_arrival_order():
    w = synth.make_workload(4, 50)
    base, _, _ = oracle.gather(w)
    rng = np.random.default_rng(21)
    by_tok = {}
    fs, fl, rf, tok = oracle.reassemble(w)
    for k, t in enumerate(tok):
        by_tok[int(t)] = base[int(np.sum(w.req_sizes[:k])):int(np.sum(w.req_sizes[:k + 1]))].copy()
    for _ in range(5):
        arr = rng.permutation(w.arrivals)
        fs2, fl2, rf2, tok2 = oracle.reassemble(w, arrivals=arr)
        assert sorted(tok2.tolist()) == sorted(tok.tolist())
        ring = w.ring.reshape(w.n_slots, w.slot_size)
        for k, t in enumerate(tok2):
            got = np.concatenate([ring[s, 58:58 + l] for s, l in zip(fs2[rf2[k]:rf2[k + 1]], fl2[rf2[k]:rf2[k + 1]])])
            assert np.array_equal(got, by_tok[int(t)])


def test_token_zero_packets_are_dropped():
    w = synth.make_custom([3000, 100], [10, 10], seed=3)
    ring = w.ring.reshape(w.n_slots, w.slot_size)
    victim = int(w.frag_slot[0])
    ring[victim, 42:50] = 0
    fs, fl, rf, tok = oracle.reassemble(w)
    assert victim not in fs.tolist() and len(tok) == 1  # the mutilated request never completes


# ---------------------------------------------------------------- batch composites vs brute force

def _py_gather(w, cap=None, cursor=0):
    ring = w.ring.reshape(w.n_slots, w.slot_size)
    hl = synth.hdr_len(w.profile)
    streams = []
    for r in range(w.n_req):
        parts = [ring[w.frag_slot[f], hl:hl + w.frag_len[f]] for f in range(w.req_first[r], w.req_first[r + 1])]
        streams.append(np.concatenate(parts) if parts else np.zeros(0, np.uint8))
    if w.in_tensor_sizes:
        outs, o = [], 0
        for s in w.in_tensor_sizes:
            outs.append(np.concatenate([st[o:o + s] for st in streams]))
            o += s
        return outs, None
    cap = cap or max(sum(len(s) for s in streams), 1)
    arena = np.zeros(cap, np.uint8)
    offs, off = [], cursor % cap
    for st in streams:
        offs.append(off)
        for k, b in enumerate(st):
            arena[(off + k) % cap] = b
        off = (off + len(st)) % cap
    offs.append(off)
    return arena, offs


@pytest.mark.parametrize("cfg,n", [(1, 5), (2, 1), (3, 9), (4, 25), (5, 1)])
def test_gather_composite_against_brute_force(cfg, n):
    w = synth.make_workload(cfg, n)
    got, offs, _ = oracle.gather(w)
    want, woffs = _py_gather(w)
    if w.in_tensor_sizes:
        for g, e in zip(got, want):
            assert np.array_equal(g, e)
    else:
        assert np.array_equal(got, want) and offs.tolist() == woffs
        assert np.array_equal(got, w.req_payload)


def test_gather_composite_wraps_like_a_mirrored_arena():
    w = synth.make_custom([3000, 5000, 700, 4100], [1, 1, 1, 1], seed=5)
    cap = 6000
    got, offs, cur = oracle.gather(w, arena_cap=cap, cursor=4500)
    want, woffs = _py_gather(w, cap=cap, cursor=4500)
    assert np.array_equal(got, want) and offs.tolist() == woffs and cur == woffs[-1]


def test_header_length_source_is_equivalent():
    w = synth.make_workload(4, 30)
    a, _, _ = oracle.gather(w, use_frag_len=True)
    b, _, _ = oracle.gather(w, use_frag_len=False)
    assert np.array_equal(a, b)


def _py_scatter(w, rx, tx0, streams, flags):
    """Brute force of one scatter pass in big-endian arithmetic."""
    hl = synth.hdr_len(w.profile)
    rxr = rx.reshape(w.n_slots, w.slot_size)
    tx = tx0.copy().reshape(w.tx_n_slots, w.slot_size)
    for r in range(w.n_req):
        st = streams[r]
        lens = synth.frame_lens(len(st), w.mtu)
        nf = len(lens)
        for i in range(nf):
            f = int(w.resp_first[r]) + i
            h = bytearray(rxr[w.hdr_src_slot[f], :hl].tobytes())
            out = bytearray(h)
            out[0:6], out[6:12] = h[6:12], h[0:6]
            out[26:30], out[30:34] = h[30:34], h[26:30]
            out[34:36], out[36:38] = h[36:38], h[34:36]
            ln = int(lens[i])
            if w.profile == synth.HDR_BL58:
                out[50:52] = i.to_bytes(2, "little")
                out[52:54] = nf.to_bytes(2, "little")
                out[54:58] = ln.to_bytes(4, "little")
            else:
                out[50:54] = b"\0\0\0\0"
                out[58:60] = i.to_bytes(2, "little")
            Lx = (hl - 42) + ln
            out[16:18] = (28 + Lx).to_bytes(2, "big")
            out[38:40] = (8 + Lx).to_bytes(2, "big")
            out[24:26] = b"\0\0"
            out[40:42] = b"\0\0"
            payload = bytes(st[i * w.mtu:i * w.mtu + ln])
            if flags & synth.F_UDP_CSUM_PSEUDO:
                sub = 16 if flags & synth.F_REF_QUIRKS else 20
                psd = bytes(out[26:34]) + bytes([0, out[23]]) + ((28 + Lx - sub) & 0xFFFF).to_bytes(2, "big")
                out[40:42] = be_sum(psd).to_bytes(2, "big")
            if flags & synth.F_IPV4_CSUM:
                out[24:26] = ((~be_sum(out[14:34])) & 0xFFFF).to_bytes(2, "big")
            if flags & synth.F_UDP_CSUM_FULL:
                out[40:42] = b"\0\0"
                psd = bytes(out[26:34]) + bytes([0, out[23]]) + (8 + Lx).to_bytes(2, "big")
                c = (~be_sum(psd + bytes(out[34:hl]) + payload + (b"\0" if ln & 1 else b""))) & 0xFFFF
                out[40:42] = (c or 0xFFFF).to_bytes(2, "big")
            slot = tx[w.tx_slot[f]]
            slot[:hl] = np.frombuffer(bytes(out), np.uint8)
            slot[hl:hl + ln] = np.frombuffer(payload, np.uint8)
    return tx.reshape(-1)


@pytest.mark.parametrize("profile", [synth.HDR_BL58, synth.HDR_REF64], ids=["bl58", "ref64"])
@pytest.mark.parametrize("cfg,n", [(1, 5), (2, 2), (3, 6), (5, 1)])
@pytest.mark.parametrize("extra", [0, synth.F_REF_QUIRKS, synth.F_IPV4_CSUM | synth.F_UDP_CSUM_FULL])
def test_scatter_composite_against_brute_force(cfg, n, extra, profile):
    w = synth.make_workload(cfg, n, profile=profile)
    flags = w.flags | extra
    per = w.resp_payload.size // w.n_req
    streams = [w.resp_payload[r * per:(r + 1) * per] for r in range(w.n_req)]
    tx = w.tx_ring_init.copy()
    if w.out_tensor_sizes:
        src = [w.resp_payload.copy()]
    else:
        src = w.resp_payload
    oracle.scatter(w, w.ring, tx, src, flags=flags)
    want = _py_scatter(w, w.ring, w.tx_ring_init, streams, flags)
    assert np.array_equal(tx, want)


def test_scatter_in_place_echo_round_trip():
    """Echo (lib_loadgen/echo_client.cc:11-32): what comes back is what went in."""
    w = synth.make_workload(4, 40)
    arena, _, _ = oracle.gather(w)
    ring = w.ring.copy()
    oracle.scatter(w, ring, ring, arena)
    w2 = synth.make_workload(4, 40)
    w2.ring = ring
    again, _, _ = oracle.gather(w2)
    assert np.array_equal(again, arena)


def test_reference_client_patterns_survive_the_path():
    """The only payload patterns the reference's own clients check:
    echo_client.cc:11-32 (DE AD BE EF cycling at every 8192nd byte, 2 elsewhere)
    and vec_add_client.cc:11-19 (MAGIC[i % 4])."""
    magic = np.array([0xDE, 0xAD, 0xBE, 0xEF], np.uint8)
    n = 20000
    echo = np.full(n, 2, np.uint8)
    echo[::8192] = magic[np.arange(len(echo[::8192])) % 4]
    vec = magic[np.arange(n) % 4]
    for pat in (echo, vec):
        w = synth.make_custom([n, n], [n, n], mtu=1024, slot_size=2048, seed=1, in_place=True)
        ring = w.ring.reshape(w.n_slots, w.slot_size)
        for r in range(2):
            for k, f in enumerate(range(w.req_first[r], w.req_first[r + 1])):
                ln = int(w.frag_len[f])
                ring[w.frag_slot[f], 58:58 + ln] = pat[k * 1024:k * 1024 + ln]
        arena, _, _ = oracle.gather(w)
        assert np.array_equal(arena, np.concatenate([pat, pat]))
        rr = w.ring.copy()
        oracle.scatter(w, rr, rr, arena)
        assert np.array_equal(rr.reshape(w.n_slots, w.slot_size)[:, 58:], ring[:, 58:])


# ---------------------------------------------------------------- golden digests

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "digests.json")


def test_golden_digests():
    """Digests written by tests/golden/make_golden.py in the container that
    holds the reference tree; they keep the oracle from drifting afterwards."""
    from golden.make_golden import digests
    with open(GOLDEN) as f:
        want = json.load(f)
    got = digests()
    assert got == want


def test_c_abi_exports_every_declared_symbol():
    import re
    from splitrpc_amd import capi
    hdr = open(os.path.join(os.path.dirname(os.path.dirname(__file__)), "include", "sg_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(sg_hip_\w+)\s*\(", hdr)) - {"sg_hip_cfg", "sg_hip_ctx"})
    lib = C.CDLL(capi.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert sorted(capi.SYMBOLS) == declared
    assert lib.sg_hip_abi_version() == 3
