"""ctypes bindings of the C ABI declared in ``include/sg_hip.h``.

The library is loaded from ``splitrpc_amd/libsg_hip.so`` (built in-tree by
``python -m splitrpc_amd.build``).  There is no fallback: if the library is
missing or a symbol is absent, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsg_hip.so")

SG_OK = 0
SG_E_INVAL = -22
SG_E_NOMEM = -12
SG_E_HIP = -5
SG_E_DATA = -74

HDR_BL58 = 0
HDR_REF64 = 1

F_IPV4_CSUM = 1 << 0
F_UDP_CSUM_PSEUDO = 1 << 1
F_UDP_CSUM_FULL = 1 << 2
F_REF_QUIRKS = 1 << 3
F_RULE_FRAGS = 1 << 4
F_NO_FUSE = 1 << 5
F_REUSE_DESC = 1 << 6
F_ASYNC = 1 << 16
F_NO_XCD_REMAP = 1 << 17
F_NO_SMALL = 1 << 18
F_FORCE_SMALL = 1 << 19
F_SELF_ADVANCE = 1 << 20
F_TAIL_KERNEL = 1 << 21
F_SMALL_GROUPS = 1 << 22

ABI_VERSION = 3  # SG_HIP_ABI_VERSION of include/sg_hip.h these mirrors were written against
MAX_BI_SIZE = 1024
MAX_TENSORS = 4

# every symbol include/sg_hip.h declares
SYMBOLS = [
    "sg_hip_create", "sg_hip_destroy", "sg_hip_last_error", "sg_hip_abi_version", "sg_hip_stream",
    "sg_hip_sync", "sg_hip_gather", "sg_hip_scatter", "sg_hip_swap_hdrs", "sg_hip_set_hdrs", "sg_hip_gather_batch",
    "sg_hip_scatter_batch", "sg_hip_reassemble", "sg_hip_set_cursor", "sg_hip_get_cursor", "sg_hip_set_profiling",
    "sg_hip_kernel_time", "sg_hip_gather_batch_static", "sg_hip_reassemble_reset", "sg_hip_reassemble_evict",
    "sg_hip_set_slot_index", "sg_hip_get_slot_index", "sg_hip_shunt_batch", "sg_hip_pack_tables", "sg_hip_stream_queue",
]

SLOT_FREE, SLOT_RX_COMPLETE, SLOT_WORK_COMPLETE, SLOT_TX_COMPLETE = 0, 1, 2, 3

STATIC_MAX_REQS = 4096
STATIC_MAX_FRAMES = 65536


class HBufs(C.Structure):
    _pack_ = 1
    _fields_ = [("burst_items", C.c_uint64 * MAX_BI_SIZE), ("num_items", C.c_uint16)]


class SkBuf(C.Structure):
    _pack_ = 1
    _fields_ = [("i_buf", C.c_uint64 * MAX_BI_SIZE), ("o_buf", C.c_uint64 * MAX_BI_SIZE),
                ("len", C.c_uint64 * (MAX_BI_SIZE - 1)), ("num_items", C.c_uint64)]


class Cfg(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("max_reqs", C.c_uint32), ("max_frames", C.c_uint32),
                ("flags", C.c_uint32), ("stream", C.c_void_p)]


class RingDesc(C.Structure):
    _fields_ = [("base", C.c_void_p), ("n_slots", C.c_uint32), ("slot_size", C.c_uint32),
                ("hdr_profile", C.c_uint32), ("reserved", C.c_uint32)]


class AppDesc(C.Structure):
    _fields_ = [("tensor_base", C.c_void_p * MAX_TENSORS), ("tensor_size", C.c_uint64 * MAX_TENSORS),
                ("n_tensors", C.c_uint32), ("arena_mirrored", C.c_uint32), ("arena", C.c_void_p),
                ("arena_cap", C.c_uint64)]


class GatherArgs(C.Structure):
    _fields_ = [("ring", RingDesc), ("frag_slot", C.c_void_p), ("frag_len", C.c_void_p),
                ("req_first", C.c_void_p), ("n_req", C.c_uint32), ("n_frags", C.c_uint32),
                ("app", AppDesc), ("offsets_out", C.c_void_p), ("flags", C.c_uint32),
                ("mtu", C.c_uint32), ("fixed_req_size", C.c_uint64), ("counts", C.c_void_p),
                ("slot_state", C.c_void_p), ("n_slot_states", C.c_uint32), ("reserved2", C.c_uint32)]


class ScatterArgs(C.Structure):
    _fields_ = [("rx", RingDesc), ("tx", RingDesc), ("tx_slot", C.c_void_p),
                ("hdr_src_slot", C.c_void_p), ("resp_first", C.c_void_p), ("resp_size", C.c_void_p),
                ("fixed_resp_size", C.c_uint64), ("n_req", C.c_uint32), ("n_frames", C.c_uint32),
                ("mtu", C.c_uint32), ("flags", C.c_uint32), ("app", AppDesc),
                ("offsets_out", C.c_void_p), ("hdr_templates", C.c_void_p), ("req_token", C.c_void_p),
                ("hdr_src_req", C.c_void_p), ("counts", C.c_void_p), ("slot_state", C.c_void_p),
                ("n_slot_states", C.c_uint32), ("reserved2", C.c_uint32)]


class FragTable(C.Structure):
    _fields_ = [("off", C.c_uint32 * MAX_BI_SIZE), ("len", C.c_uint32 * MAX_BI_SIZE)]


class PackArgs(C.Structure):
    _fields_ = [("tables", C.c_void_p), ("n_tables", C.c_uint32), ("n_req", C.c_uint32), ("table_idx", C.c_void_p),
                ("req_first", C.c_void_p), ("n_frags", C.c_uint32), ("reserved", C.c_uint32),
                ("pkt_base", C.c_uint64), ("ring", RingDesc), ("frag_slot", C.c_void_p), ("frag_len", C.c_void_p),
                ("req_first_out", C.c_void_p), ("blob_src", C.c_void_p), ("blob_dst", C.c_void_p),
                ("blob_words", C.c_uint32), ("reserved2", C.c_uint32), ("stream", C.c_void_p)]


class ReassembleArgs(C.Structure):
    _fields_ = [("ring", RingDesc), ("arrivals", C.c_void_p), ("len_nic", C.c_void_p),
                ("n_arrivals", C.c_uint32), ("flags", C.c_uint32), ("req_size", C.c_uint64),
                ("frag_slot", C.c_void_p), ("frag_len", C.c_void_p), ("req_first", C.c_void_p),
                ("req_token", C.c_void_p), ("req_hdr_slot", C.c_void_p), ("counts_out", C.c_void_p),
                ("n_arrivals_dev", C.c_void_p)]


_lib = None


def load() -> C.CDLL:
    """Load the HIP library; raise if it is not built or lacks a symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m splitrpc_amd.build` "
            "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    missing = [s for s in SYMBOLS if not hasattr(lib, s)]
    if missing:
        raise RuntimeError(f"{LIB_PATH} lacks symbols {missing}")
    P = C.c_void_p
    lib.sg_hip_create.argtypes = [C.c_int, C.POINTER(Cfg)]
    lib.sg_hip_create.restype = P
    lib.sg_hip_destroy.argtypes = [P]
    lib.sg_hip_destroy.restype = None
    lib.sg_hip_last_error.argtypes = [P]
    lib.sg_hip_last_error.restype = C.c_char_p
    lib.sg_hip_abi_version.restype = C.c_int
    if lib.sg_hip_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} speaks ABI version {lib.sg_hip_abi_version()}, this module {ABI_VERSION}: "
                           "rebuild with `python -m splitrpc_amd.build`")
    lib.sg_hip_stream.argtypes = [P]
    lib.sg_hip_stream.restype = P
    lib.sg_hip_sync.argtypes = [P]
    lib.sg_hip_gather.argtypes = [P, C.POINTER(SkBuf)]
    lib.sg_hip_scatter.argtypes = [P, C.POINTER(SkBuf)]
    lib.sg_hip_swap_hdrs.argtypes = [P, C.POINTER(HBufs), C.c_uint32, C.c_uint64, C.c_uint32, C.c_uint32]
    lib.sg_hip_set_hdrs.argtypes = [P, C.POINTER(HBufs), C.c_void_p, C.c_uint64, C.c_uint32, C.c_uint64,
                                    C.c_uint32, C.c_uint32]
    lib.sg_hip_gather_batch.argtypes = [P, C.POINTER(GatherArgs)]
    lib.sg_hip_scatter_batch.argtypes = [P, C.POINTER(ScatterArgs)]
    lib.sg_hip_shunt_batch.argtypes = [P, C.POINTER(GatherArgs), C.POINTER(ScatterArgs)]
    lib.sg_hip_stream_queue.argtypes = [P, P, C.POINTER(C.c_uint64)]
    lib.sg_hip_pack_tables.argtypes = [P, C.POINTER(PackArgs)]
    lib.sg_hip_gather_batch_static.argtypes = [C.c_int, P, C.POINTER(GatherArgs), P, P]
    lib.sg_hip_reassemble.argtypes = [P, C.POINTER(ReassembleArgs), C.POINTER(C.c_uint32 * 4)]
    lib.sg_hip_reassemble_reset.argtypes = [P]
    lib.sg_hip_reassemble_evict.argtypes = [P, C.c_uint32, C.POINTER(C.c_uint32)]
    lib.sg_hip_set_slot_index.argtypes = [P, C.c_int, C.c_uint32]
    lib.sg_hip_get_slot_index.argtypes = [P, C.c_int, C.POINTER(C.c_uint32)]
    lib.sg_hip_set_cursor.argtypes = [P, C.c_int, C.c_uint64]
    lib.sg_hip_get_cursor.argtypes = [P, C.c_int, C.POINTER(C.c_uint64)]
    lib.sg_hip_set_profiling.argtypes = [P, C.c_int]
    lib.sg_hip_kernel_time.argtypes = [P, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_uint64)]
    _lib = lib
    return lib
