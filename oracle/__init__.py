"""ctypes face of the CPU oracle (oracle/sg_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke`` and
by the CPU-baseline leg of ``bench.py`` as the checker.  The shipped package
never imports it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsg_oracle.so")
REF_PATH = os.path.join(_HERE, "_ref", "libsg_ref.so")

MAX_BI_SIZE = 1024
MAX_TENSORS = 4


def build(force: bool = False) -> None:
    """Compile the oracle (and the reference probe where the reference tree exists)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


class Ring(C.Structure):
    _fields_ = [("base", C.c_void_p), ("n_slots", C.c_uint32), ("slot_size", C.c_uint32),
                ("profile", C.c_uint32)]


class AppBufs(C.Structure):
    _fields_ = [("base", C.c_void_p * MAX_TENSORS), ("size", C.c_uint64 * MAX_TENSORS),
                ("n_tensors", C.c_uint32), ("arena", C.c_void_p), ("arena_cap", C.c_uint64)]


class HBufs(C.Structure):
    _pack_ = 1
    _fields_ = [("burst_items", C.c_uint64 * MAX_BI_SIZE), ("num_items", C.c_uint16)]


class Bufs(C.Structure):
    _pack_ = 1
    _fields_ = [("burst_items", C.c_uint64 * MAX_BI_SIZE), ("item_size", C.c_uint64 * MAX_BI_SIZE),
                ("num_items", C.c_uint16)]


class SkBuf(C.Structure):
    _pack_ = 1
    _fields_ = [("i_buf", C.c_uint64 * MAX_BI_SIZE), ("o_buf", C.c_uint64 * MAX_BI_SIZE),
                ("len", C.c_uint64 * (MAX_BI_SIZE - 1)), ("num_items", C.c_uint64)]


class Tring(C.Structure):
    _fields_ = [("base", C.c_uint64), ("capacity", C.c_uint64), ("prev_offset", C.c_uint64),
                ("prev_addr", C.c_uint64)]


_lib = None
_ref = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        u8p, u32p, u64p = C.c_void_p, C.c_void_p, C.c_void_p
        L.sgo_swap_eth_hdr.argtypes = [u8p]
        L.sgo_add_ip_udp_len.argtypes = [u8p, C.c_uint16]
        L.sgo_ipv4_pseudo_csum.argtypes = [u8p, C.c_int]
        L.sgo_ipv4_pseudo_csum.restype = C.c_uint16
        L.sgo_add_udp_cksum.argtypes = [u8p, C.c_int]
        L.sgo_set_sockperf_header.argtypes = [u8p]
        L.sgo_set_conn_info.argtypes = [u8p, u8p, C.c_uint32]
        L.sgo_ipv4_hdr_csum.argtypes = [u8p]
        L.sgo_ipv4_hdr_csum.restype = C.c_uint16
        L.sgo_udp_full_csum.argtypes = [u8p, u8p]
        L.sgo_udp_full_csum.restype = C.c_uint16
        L.sgo_gen_hdr_template.argtypes = [u8p, u8p, u8p, C.c_uint32, C.c_uint32, C.c_int, C.c_int]
        L.sgo_rewrite_resp_hdr.argtypes = [u8p, C.c_uint32, C.c_uint32, C.c_uint16, C.c_uint16, C.c_uint32]
        L.sgo_template_resp_hdr.argtypes = [u8p, u8p, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint16,
                                            C.c_uint16, C.c_uint32]
        L.sgo_gather_skbs.argtypes = [C.POINTER(SkBuf), C.POINTER(Bufs), C.c_uint64]
        L.sgo_scatter_skbs.argtypes = [C.POINTER(SkBuf), C.POINTER(Bufs), C.c_uint64]
        L.sgo_sg_on_cpu.argtypes = [C.POINTER(SkBuf)]
        L.sgo_num_frames.argtypes = [C.c_uint64, C.c_uint32]
        L.sgo_num_frames.restype = C.c_uint32
        L.sgo_frame_len.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32]
        L.sgo_frame_len.restype = C.c_uint32
        L.sgo_tring_init.argtypes = [C.POINTER(Tring), C.c_uint64, C.c_uint64]
        L.sgo_tring_get_next.argtypes = [C.POINTER(Tring), C.c_uint64]
        L.sgo_tring_get_next.restype = C.c_uint64
        L.sgo_reassemble.argtypes = [C.POINTER(Ring), u32p, C.c_uint32, u32p, C.c_uint64, u32p, u32p,
                                     u32p, u64p, C.c_uint32, C.c_uint32]
        L.sgo_reassemble.restype = C.c_int64
        L.sgo_gather_batch.argtypes = [C.POINTER(Ring), u32p, u32p, u32p, C.c_uint32,
                                       C.POINTER(AppBufs), u64p, u64p]
        L.sgo_gather_batch.restype = C.c_int64
        L.sgo_scatter_batch.argtypes = [C.POINTER(Ring), C.POINTER(Ring), u32p, u32p, u32p, u64p,
                                        C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32,
                                        C.POINTER(AppBufs), u64p, u64p, u8p, u64p]
        L.sgo_scatter_batch.restype = C.c_int64
        L.sgo_now_sec.restype = C.c_double
        _lib = L
    return _lib


def ref() -> Optional[C.CDLL]:
    """The probe over the reference's own headers, or None where it was not built."""
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        R = C.CDLL(REF_PATH)
        R.ref_layout.argtypes = [C.c_int]
        R.ref_layout.restype = C.c_uint64
        R.ref_ipv4_pseudo_csum.argtypes = [C.c_void_p, C.c_uint8]
        R.ref_ipv4_pseudo_csum.restype = C.c_uint16
        R.ref_ip_nibbles.argtypes = [C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        R.ref_gen_hdr_template.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32,
                                           C.c_int, C.c_int]
        R.ref_tring_replay.argtypes = [C.c_uint64, C.c_uint64, C.c_void_p, C.c_uint32, C.c_void_p]
        _ref = R
    return _ref


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _ring(buf: np.ndarray, n_slots: int, slot_size: int, profile: int) -> Ring:
    assert buf.dtype == np.uint8 and buf.flags["C_CONTIGUOUS"] and buf.size >= n_slots * slot_size
    return Ring(buf.ctypes.data, n_slots, slot_size, profile)


def _app(tensor_sizes, tensors, arena: Optional[np.ndarray], cap: int) -> AppBufs:
    a = AppBufs()
    a.n_tensors = len(tensor_sizes)
    for i, (s, t) in enumerate(zip(tensor_sizes, tensors)):
        a.base[i] = t.ctypes.data
        a.size[i] = int(s)
    a.arena = arena.ctypes.data if arena is not None else None
    a.arena_cap = cap
    return a


def gather(w, arena_cap: Optional[int] = None, cursor: int = 0, use_frag_len: bool = True,
           out=None):
    """Run the CPU gather composite on workload ``w``.

    Packed mode returns (arena bytes, offsets[n_req+1], cursor_after);
    tensor-major mode returns (list of tensors, None, cursor).  ``out`` reuses
    a destination (arena array or tensor list) instead of allocating one."""
    L = lib()
    ring = _ring(w.ring, w.n_slots, w.slot_size, w.profile)
    fl = np.ascontiguousarray(w.frag_len, dtype=np.uint32) if use_frag_len else None
    fs = np.ascontiguousarray(w.frag_slot, dtype=np.uint32)
    rf = np.ascontiguousarray(w.req_first, dtype=np.uint32)
    cur = np.array([cursor], dtype=np.uint64)
    if w.in_tensor_sizes:
        tensors = out if out is not None else [np.zeros(w.n_req * s, dtype=np.uint8)
                                               for s in w.in_tensor_sizes]
        app = _app(w.in_tensor_sizes, tensors, None, 0)
        rc = L.sgo_gather_batch(C.byref(ring), _p(fs), _p(fl), _p(rf), w.n_req, C.byref(app), _p(cur), None)
        assert rc >= 0
        return tensors, None, int(cur[0])
    cap = int(arena_cap if arena_cap is not None else max(int(w.req_sizes.sum()), 1))
    arena = out if out is not None else np.zeros(cap, dtype=np.uint8)
    offs = np.zeros(w.n_req + 1, dtype=np.uint64)
    app = _app([], [], arena, cap)
    rc = L.sgo_gather_batch(C.byref(ring), _p(fs), _p(fl), _p(rf), w.n_req, C.byref(app), _p(cur), _p(offs))
    assert rc >= 0
    return arena, offs, int(cur[0])


def scatter(w, rx_ring: np.ndarray, tx_ring: np.ndarray, resp_src, arena_cap: Optional[int] = None,
            cursor: int = 0, flags: Optional[int] = None, fixed_size: Optional[int] = None,
            templates: Optional[np.ndarray] = None, tokens: Optional[np.ndarray] = None):
    """Run the CPU scatter composite.  ``tx_ring`` is modified in place (pass
    ``rx_ring`` itself for in-place responses).  ``resp_src`` is the packed
    arena (uint8 array) or the list of tensor-major output tensors.
    ``templates`` (n_req x 64 uint8) switches the headers to the template
    path, with ``tokens`` (n_req uint64) as the request tokens."""
    L = lib()
    rx = _ring(rx_ring, w.n_slots, w.slot_size, w.profile)
    tx = _ring(tx_ring, w.tx_n_slots, w.slot_size, w.profile)
    ts = np.ascontiguousarray(w.tx_slot, dtype=np.uint32)
    hs = np.ascontiguousarray(w.hdr_src_slot, dtype=np.uint32)
    rf = np.ascontiguousarray(w.resp_first, dtype=np.uint32)
    rs = None if fixed_size is not None else np.ascontiguousarray(w.resp_sizes, dtype=np.uint64)
    cur = np.array([cursor], dtype=np.uint64)
    offs = np.zeros(w.n_req + 1, dtype=np.uint64)
    tm = None if templates is None else np.ascontiguousarray(templates, dtype=np.uint8)
    tk = None if tokens is None else np.ascontiguousarray(tokens, dtype=np.uint64)
    assert tm is None or tm.size == w.n_req * 64
    if w.out_tensor_sizes:
        app = _app(w.out_tensor_sizes, resp_src, None, 0)
    else:
        cap = int(arena_cap if arena_cap is not None else resp_src.size)
        app = _app([], [], resp_src, cap)
    rc = L.sgo_scatter_batch(C.byref(rx), C.byref(tx), _p(ts), _p(hs), _p(rf), _p(rs),
                             int(fixed_size or 0), w.n_req, w.mtu,
                             w.flags if flags is None else flags, C.byref(app), _p(cur), _p(offs),
                             _p(tm), _p(tk))
    assert rc >= 0, "oracle scatter rejected the tables"
    return offs, int(cur[0])


def reassemble(w, arrivals: Optional[np.ndarray] = None, req_size: int = 0,
               frag_len_nic: Optional[np.ndarray] = None) -> Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]:
    L = lib()
    ring = _ring(w.ring, w.n_slots, w.slot_size, w.profile)
    arr = np.ascontiguousarray(w.arrivals if arrivals is None else arrivals, dtype=np.uint32)
    max_req, max_frag = len(arr) + 1, len(arr) + 1
    fs = np.zeros(max_frag, np.uint32)
    fl = np.zeros(max_frag, np.uint32)
    rf = np.zeros(max_req + 1, np.uint32)
    tok = np.zeros(max_req, np.uint64)
    n = L.sgo_reassemble(C.byref(ring), _p(arr), len(arr), _p(frag_len_nic), req_size, _p(fs), _p(fl),
                         _p(rf), _p(tok), max_req, max_frag)
    assert n >= 0
    nf = int(rf[n])
    return fs[:nf], fl[:nf], rf[: n + 1], tok[:n]
