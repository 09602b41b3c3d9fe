"""Thin Python face of the C ABI for tests, the smoke check and the benchmark.

torch is used for device memory and streams only; every operation goes through
``libsg_hip.so``.  Tables are int32 / int64 tensors holding the bit patterns of
the ABI's uint32 / uint64 arrays.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from . import capi
from .synth import Workload


class SgError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"sg_hip error {code}: {msg}")
        self.code = code


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def to_dev(a: np.ndarray, device) -> torch.Tensor:
    """Upload a numpy array, keeping its bits (uint32 -> int32, uint64 -> int64)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    elif a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(a.copy()).to(device)


@dataclass
class RingRef:
    buf: torch.Tensor  # uint8
    n_slots: int
    slot_size: int
    profile: int

    def desc(self) -> capi.RingDesc:
        assert self.buf.dtype == torch.uint8 and self.buf.is_contiguous()
        assert self.buf.numel() >= self.n_slots * self.slot_size
        return capi.RingDesc(self.buf.data_ptr(), self.n_slots, self.slot_size, self.profile, 0)


@dataclass
class AppRef:
    """Packed arena (``arena``, ``cap``) or tensor-major buffers (``tensors`` with
    per-request ``sizes``)."""
    arena: Optional[torch.Tensor] = None
    cap: int = 0
    mirrored: bool = False
    tensors: Sequence[torch.Tensor] = ()
    sizes: Sequence[int] = ()
    arena_ptr: int = 0   # raw device address instead of ``arena`` (memory torch does not own)

    def desc(self) -> capi.AppDesc:
        d = capi.AppDesc()
        d.n_tensors = len(self.tensors)
        for i, (t, s) in enumerate(zip(self.tensors, self.sizes)):
            d.tensor_base[i] = t.data_ptr()
            d.tensor_size[i] = int(s)
        if self.arena is not None:
            d.arena = self.arena.data_ptr()
            d.arena_cap = int(self.cap)
        elif self.arena_ptr:
            d.arena = self.arena_ptr
            d.arena_cap = int(self.cap)
        d.arena_mirrored = 1 if self.mirrored else 0
        return d


class SgContext:
    def __init__(self, device: int = 0, max_reqs: int = 4096, max_frames: int = 65536,
                 stream: Optional[int] = None):
        self.lib = capi.load()
        cfg = capi.Cfg(C.sizeof(capi.Cfg), max_reqs, max_frames, 0, stream)
        self.h = self.lib.sg_hip_create(device, C.byref(cfg))
        if not self.h:
            raise SgError(capi.SG_E_HIP, self.lib.sg_hip_last_error(None).decode())
        self.device = device

    def close(self) -> None:
        if getattr(self, "h", None):
            self.lib.sg_hip_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _after_torch() -> None:
        """The context launches on its own non-blocking stream: what torch has
        queued on its stream (fills, uploads, copies of test data) must be done
        before a kernel of this library reads or overwrites the same memory."""
        torch.cuda.current_stream().synchronize()

    def _check(self, rc: int) -> None:
        if rc != capi.SG_OK:
            raise SgError(rc, self.lib.sg_hip_last_error(self.h).decode())

    @property
    def stream(self) -> int:
        return int(self.lib.sg_hip_stream(self.h) or 0)

    def sync(self) -> None:
        self._check(self.lib.sg_hip_sync(self.h))

    def stream_queue(self, stream: Optional[int] = None) -> int:
        """Address of the hardware queue the context's stream (or ``stream``)
        dispatches to: streams that share one run their kernels one after the
        other."""
        q = C.c_uint64(0)
        self._check(self.lib.sg_hip_stream_queue(self.h, C.c_void_p(stream) if stream else None, C.byref(q)))
        return int(q.value)

    @classmethod
    def apart_from(cls, others: Sequence["SgContext"], device: int = 0, **kw) -> "SgContext":
        """A context whose stream dispatches to another hardware queue than
        those of ``others`` (the runtime deals its few hardware queues out to
        streams in turns, so two contexts made at different times may share
        one, and calls queued to them then never overlap).  Falls back to the
        last one made."""
        taken = {o.stream_queue() for o in others}
        spare, found = [], None
        for _ in range(8):
            c = cls(device, **kw)
            if c.stream_queue() not in taken:
                found = c
                break
            spare.append(c)
        if found is None:
            found = spare.pop()
        for c in spare:
            c.close()
        return found

    def set_cursor(self, which: int, value: int) -> None:
        self._check(self.lib.sg_hip_set_cursor(self.h, which, value))

    def get_cursor(self, which: int) -> int:
        v = C.c_uint64(0)
        self._check(self.lib.sg_hip_get_cursor(self.h, which, C.byref(v)))
        return int(v.value)

    def set_profiling(self, on: bool) -> None:
        self._check(self.lib.sg_hip_set_profiling(self.h, 1 if on else 0))

    def kernel_time(self, which: int):
        ms, n = C.c_double(0), C.c_uint64(0)
        self._check(self.lib.sg_hip_kernel_time(self.h, which, C.byref(ms), C.byref(n)))
        return float(ms.value), int(n.value)

    # -- batched -----------------------------------------------------------
    @staticmethod
    def gather_args(ring: RingRef, frag_slot: torch.Tensor, frag_len: Optional[torch.Tensor],
                    req_first: torch.Tensor, n_req: int, n_frags: int, app: AppRef,
                    offsets_out: Optional[torch.Tensor] = None, flags: int = 0,
                    fixed_req_size: int = 0, mtu: int = 0, counts: Optional[torch.Tensor] = None,
                    slot_state: Optional[torch.Tensor] = None) -> capi.GatherArgs:
        a = capi.GatherArgs()
        a.ring = ring.desc()
        a.frag_slot = frag_slot.data_ptr()
        a.frag_len = frag_len.data_ptr() if frag_len is not None else None
        a.req_first = req_first.data_ptr()
        a.n_req = n_req
        a.n_frags = n_frags
        a.app = app.desc()
        a.offsets_out = offsets_out.data_ptr() if offsets_out is not None else None
        a.flags = flags
        a.fixed_req_size = int(fixed_req_size)
        a.mtu = int(mtu)
        a.counts = counts.data_ptr() if counts is not None else None
        if slot_state is not None:
            a.slot_state = slot_state.data_ptr()
            a.n_slot_states = int(slot_state.numel())
        return a

    def gather_batch(self, *args, **kw) -> None:
        self.gather_batch_raw(self.gather_args(*args, **kw))

    def gather_batch_raw(self, a: capi.GatherArgs) -> None:
        if not (a.flags & capi.F_ASYNC):
            self._after_torch()
        rc = self.lib.sg_hip_gather_batch(self.h, C.byref(a))
        if rc != capi.SG_OK:
            self._check(rc)

    @staticmethod
    def scatter_args(rx: RingRef, tx: RingRef, tx_slot: torch.Tensor,
                     hdr_src_slot: torch.Tensor, resp_first: torch.Tensor,
                     resp_size: Optional[torch.Tensor], fixed_resp_size: int, n_req: int,
                     n_frames: int, mtu: int, app: AppRef,
                     offsets_out: Optional[torch.Tensor] = None, flags: int = 0,
                     hdr_templates: Optional[torch.Tensor] = None,
                     req_token: Optional[torch.Tensor] = None, hdr_src_req: Optional[torch.Tensor] = None,
                     counts: Optional[torch.Tensor] = None,
                     slot_state: Optional[torch.Tensor] = None) -> capi.ScatterArgs:
        a = capi.ScatterArgs()
        a.rx = rx.desc()
        a.tx = tx.desc()
        a.tx_slot = tx_slot.data_ptr()
        a.hdr_src_slot = hdr_src_slot.data_ptr() if hdr_src_slot is not None else None
        a.resp_first = resp_first.data_ptr()
        a.resp_size = resp_size.data_ptr() if resp_size is not None else None
        a.fixed_resp_size = int(fixed_resp_size)
        a.n_req = n_req
        a.n_frames = n_frames
        a.mtu = mtu
        a.flags = flags
        a.app = app.desc()
        a.offsets_out = offsets_out.data_ptr() if offsets_out is not None else None
        a.hdr_templates = hdr_templates.data_ptr() if hdr_templates is not None else None
        a.req_token = req_token.data_ptr() if req_token is not None else None
        a.hdr_src_req = hdr_src_req.data_ptr() if hdr_src_req is not None else None
        a.counts = counts.data_ptr() if counts is not None else None
        if slot_state is not None:
            a.slot_state = slot_state.data_ptr()
            a.n_slot_states = int(slot_state.numel())
        return a

    def scatter_batch(self, *args, **kw) -> None:
        self.scatter_batch_raw(self.scatter_args(*args, **kw))

    def scatter_batch_raw(self, a: capi.ScatterArgs) -> None:
        if not (a.flags & capi.F_ASYNC):
            self._after_torch()
        rc = self.lib.sg_hip_scatter_batch(self.h, C.byref(a))
        if rc != capi.SG_OK:
            self._check(rc)

    def shunt_batch_raw(self, g: capi.GatherArgs, s: capi.ScatterArgs) -> None:
        """One pass of the shunter's loop: gather and scatter, in one launch
        where the two calls can share one."""
        if not (g.flags & s.flags & capi.F_ASYNC):
            self._after_torch()
        rc = self.lib.sg_hip_shunt_batch(self.h, C.byref(g), C.byref(s))
        if rc != capi.SG_OK:
            self._check(rc)

    @staticmethod
    def reassemble_args(ring: RingRef, arrivals: torch.Tensor, n_arrivals: int, frag_slot: torch.Tensor,
                        frag_len: torch.Tensor, req_first: torch.Tensor, req_token: Optional[torch.Tensor] = None,
                        len_nic: Optional[torch.Tensor] = None, req_size: int = 0,
                        req_hdr_slot: Optional[torch.Tensor] = None, counts_out: Optional[torch.Tensor] = None,
                        n_arrivals_dev: Optional[torch.Tensor] = None, flags: int = 0) -> capi.ReassembleArgs:
        a = capi.ReassembleArgs()
        a.ring = ring.desc()
        a.arrivals = arrivals.data_ptr()
        a.len_nic = len_nic.data_ptr() if len_nic is not None else None
        a.n_arrivals = n_arrivals
        a.flags = flags
        a.req_size = int(req_size)
        a.frag_slot = frag_slot.data_ptr()
        a.frag_len = frag_len.data_ptr()
        a.req_first = req_first.data_ptr()
        a.req_token = req_token.data_ptr() if req_token is not None else None
        a.req_hdr_slot = req_hdr_slot.data_ptr() if req_hdr_slot is not None else None
        a.counts_out = counts_out.data_ptr() if counts_out is not None else None
        a.n_arrivals_dev = n_arrivals_dev.data_ptr() if n_arrivals_dev is not None else None
        return a

    def reassemble_raw(self, a: capi.ReassembleArgs):
        """Returns (requests completed, their fragments, arrivals dropped,
        requests still in flight); all zero for an SG_F_ASYNC call."""
        counts = (C.c_uint32 * 4)()
        if not (a.flags & capi.F_ASYNC):
            self._after_torch()
        rc = self.lib.sg_hip_reassemble(self.h, C.byref(a), C.byref(counts))
        if rc != capi.SG_OK:
            self._check(rc)
        return tuple(int(x) for x in counts)

    def reassemble(self, *args, **kw):
        """Sort a burst of arrivals into requests on the device; incomplete
        requests stay on the device for later calls.  Returns (requests
        completed, their fragments, requests still in flight)."""
        n_req, n_frag, self.last_dropped, in_flight = self.reassemble_raw(self.reassemble_args(*args, **kw))
        return n_req, n_frag, in_flight

    def reassemble_reset(self) -> None:
        self._check(self.lib.sg_hip_reassemble_reset(self.h))

    def reassemble_evict(self, max_age_calls: int) -> int:
        n = C.c_uint32(0)
        self._check(self.lib.sg_hip_reassemble_evict(self.h, max_age_calls, C.byref(n)))
        return int(n.value)

    def set_slot_index(self, which: int, value: int) -> None:
        self._check(self.lib.sg_hip_set_slot_index(self.h, which, value))

    def get_slot_index(self, which: int) -> int:
        v = C.c_uint32(0)
        self._check(self.lib.sg_hip_get_slot_index(self.h, which, C.byref(v)))
        return int(v.value)

    # -- per request ---------------------------------------------------------
    def copy_runs(self, src: Sequence[int], dst: Sequence[int], lens: Sequence[int],
                  scatter: bool = False) -> None:
        skb = capi.SkBuf()
        n = len(lens)
        assert n <= capi.MAX_BI_SIZE - 1
        for i in range(n):
            skb.i_buf[i] = src[i]
            skb.o_buf[i] = dst[i]
            skb.len[i] = lens[i]
        skb.num_items = n
        fn = self.lib.sg_hip_scatter if scatter else self.lib.sg_hip_gather
        self._after_torch()
        self._check(fn(self.h, C.byref(skb)))

    def swap_hdrs(self, hdr_ptrs: Sequence[int], profile: int, payload_size: int, mtu: int,
                  flags: int) -> None:
        hb = capi.HBufs()
        for i, p in enumerate(hdr_ptrs):
            hb.burst_items[i] = p
        hb.num_items = len(hdr_ptrs)
        self._after_torch()
        self._check(self.lib.sg_hip_swap_hdrs(self.h, C.byref(hb), profile, payload_size, mtu, flags))

    def set_hdrs(self, hdr_ptrs: Sequence[int], template: bytes, token: int, profile: int,
                 payload_size: int, mtu: int, flags: int) -> None:
        hb = capi.HBufs()
        for i, p in enumerate(hdr_ptrs):
            hb.burst_items[i] = p
        hb.num_items = len(hdr_ptrs)
        assert len(template) >= 64
        t = (C.c_uint8 * 64).from_buffer_copy(bytes(template[:64]))
        self._after_torch()
        self._check(self.lib.sg_hip_set_hdrs(self.h, C.byref(hb), t, token, profile, payload_size, mtu, flags))


class DeviceWorkload:
    """A synthetic workload staged in one GPU's memory: the landing-zone ring,
    the fragment tables and the application buffers."""

    @staticmethod
    def _shifted(t: torch.Tensor, shift: int) -> torch.Tensor:
        if not shift:
            return t
        backing = torch.zeros(t.numel() + shift + 16, dtype=t.dtype, device=t.device)
        view = backing[shift:shift + t.numel()]
        view.copy_(t)
        return view

    def __init__(self, w: Workload, device="cuda:0", arena_slack: int = 0, copies: int = 1,
                 unique_tokens: bool = False, ring_shift: int = 0):
        """``ring_shift`` moves both rings that many bytes off the allocator's
        alignment (rings only have to start at an even address).
        ``copies`` > 1 lays that many copies of the ring (and of the tables,
        slot indices shifted) side by side, so that one call moves ``copies``
        batches and the working set outgrows the caches."""
        self.w = w
        self.copies = copies
        self._args = {}
        dev = torch.device(device)
        self.dev = dev
        k = copies
        self.n_req = w.n_req * k
        self.n_frags = w.n_frags * k
        self.n_frames = w.n_resp_frames * k
        ring1 = torch.from_numpy(w.ring).to(dev)
        self.ring = ring1.repeat(k) if k > 1 else ring1
        if unique_tokens and k > 1:
            # give every copy its own request tokens (bits 40..55 of the u64 at byte 42)
            v = self.ring.view(k, w.n_slots, w.slot_size)
            c = torch.arange(k, device=dev, dtype=torch.int32).view(k, 1)
            used = torch.from_numpy(w.frag_slot.astype(np.int64)).to(dev)
            v[:, used, 47] = ((v[:, used, 47].to(torch.int32) + (c & 0xFF)) & 0xFF).to(torch.uint8)
            v[:, used, 48] = ((v[:, used, 48].to(torch.int32) + (c >> 8)) & 0xFF).to(torch.uint8)
        self.ring = self._shifted(self.ring, ring_shift)
        self.rx = RingRef(self.ring, w.n_slots * k, w.slot_size, w.profile)

        def tile_slots(a: np.ndarray, n_slots: int) -> np.ndarray:
            return np.concatenate([a.astype(np.uint32) + np.uint32(i * n_slots) for i in range(k)])

        def tile_csr(first: np.ndarray) -> np.ndarray:
            body = [first[:-1].astype(np.uint32) + np.uint32(i * int(first[-1])) for i in range(k)]
            return np.concatenate(body + [np.array([int(first[-1]) * k], dtype=np.uint32)])

        self.arrivals = to_dev(tile_slots(w.arrivals, w.n_slots), dev)
        self.frag_slot = to_dev(tile_slots(w.frag_slot, w.n_slots), dev)
        self.frag_len = to_dev(np.tile(w.frag_len, k), dev)
        self.req_first = to_dev(tile_csr(w.req_first), dev)
        self.tx_slot = to_dev(tile_slots(w.tx_slot, w.tx_n_slots), dev)
        self.hdr_src_slot = to_dev(tile_slots(w.hdr_src_slot, w.n_slots), dev)
        self.resp_first = to_dev(tile_csr(w.resp_first), dev)
        self.resp_size = to_dev(np.tile(w.resp_sizes, k), dev)
        if w.tx_in_place:
            self.tx_ring = self.ring
        else:
            t1 = torch.from_numpy(w.tx_ring_init).to(dev)
            self.tx_ring = self._shifted(t1.repeat(k) if k > 1 else t1, ring_shift)
        self.tx = RingRef(self.tx_ring, w.tx_n_slots * k, w.slot_size, w.profile)

        # request side application buffers
        if w.in_tensor_sizes:
            self.in_tensors = [torch.zeros(self.n_req * s, dtype=torch.uint8, device=dev)
                               for s in w.in_tensor_sizes]
            self.req_app = AppRef(tensors=self.in_tensors, sizes=w.in_tensor_sizes)
            self.req_offsets = None
        else:
            cap = int(w.req_sizes.sum()) * k + arena_slack
            self.req_arena = torch.zeros(max(cap, 16), dtype=torch.uint8, device=dev)
            self.req_app = AppRef(arena=self.req_arena, cap=max(cap, 16))
            self.req_offsets = torch.zeros(self.n_req + 1, dtype=torch.int64, device=dev)
        # response side
        resp1 = torch.from_numpy(w.resp_payload).to(dev)
        if w.out_tensor_sizes:
            assert len(w.out_tensor_sizes) == 1 or True
            # responses concatenated in batch order are tensor-major already when there is one tensor
            self.out_tensors = self._split_outputs(w, k, dev)
            self.resp_app = AppRef(tensors=self.out_tensors, sizes=w.out_tensor_sizes)
            self.resp_offsets = None
        elif w.tx_in_place:
            # echo: responses are read from where gather put the requests
            self.resp_app = self.req_app
            self.resp_offsets = torch.zeros(self.n_req + 1, dtype=torch.int64, device=dev)
        else:
            self.resp_arena = resp1.repeat(k) if k > 1 else resp1
            cap = int(self.resp_arena.numel())
            if cap < 16:
                self.resp_arena = torch.zeros(16, dtype=torch.uint8, device=dev)
            self.resp_app = AppRef(arena=self.resp_arena, cap=max(cap, 16))
            self.resp_offsets = torch.zeros(self.n_req + 1, dtype=torch.int64, device=dev)

    @staticmethod
    def _split_outputs(w: Workload, k: int, dev) -> List[torch.Tensor]:
        per_req = int(sum(w.out_tensor_sizes))
        rp = w.resp_payload.reshape(w.n_req, per_req)
        outs, o = [], 0
        for s in w.out_tensor_sizes:
            t = torch.from_numpy(np.ascontiguousarray(rp[:, o:o + s]).reshape(-1)).to(dev)
            outs.append(t.repeat(k) if k > 1 else t)
            o += s
        return outs

    def gather_call(self, ctx: SgContext, flags: int = 0, use_frag_len: bool = False,
                    fixed: bool = True, rule: bool = False) -> capi.GatherArgs:
        """The argument block of this workload's gather call (built once per
        combination and kept).  ``fixed``: declare the common request size when
        all requests have one (offsets are then multiples of it instead of a
        prefix scan).  ``rule``: also state that fragments follow the
        fragmenting rule, which lets the copy kernel work without a descriptor
        pass."""
        key = ("g", use_frag_len, fixed, rule)
        a = self._args.get(key)
        if a is None:
            need_len = use_frag_len or self.w.profile != 0
            sizes = self.w.req_sizes
            fx = int(sizes[0]) if fixed and len(sizes) and bool((sizes == sizes[0]).all()) else 0
            a = ctx.gather_args(self.rx, self.frag_slot, self.frag_len if need_len else None,
                                self.req_first, self.n_req, self.n_frags, self.req_app,
                                self.req_offsets, 0, fixed_req_size=fx, mtu=self.w.mtu)
            a._base_flags = capi.F_RULE_FRAGS if (rule and fx) else 0
            self._args[key] = a
        a.flags = flags | a._base_flags
        self._described = not (a._base_flags & capi.F_RULE_FRAGS)  # a descriptor pass runs
        return a

    def gather(self, ctx: SgContext, flags: int = 0, use_frag_len: bool = False,
               fixed: bool = True, rule: bool = False) -> None:
        ctx.gather_batch_raw(self.gather_call(ctx, flags, use_frag_len, fixed, rule))

    def scatter_call(self, ctx: SgContext, flags: int = 0, fixed: bool = True, fuse: bool = True,
                     templates: Optional[torch.Tensor] = None, tokens: Optional[torch.Tensor] = None,
                     reuse: bool = False) -> capi.ScatterArgs:
        """The argument block of this workload's scatter call.  ``templates``
        (n_req x 64 uint8 on the device) takes the frame headers from
        connection templates instead of request headers.  ``reuse``: an echo
        answered in place right after this workload's gather reuses that call's
        descriptors where it ran a descriptor pass."""
        if not fuse:
            flags |= capi.F_NO_FUSE
        if reuse and self.w.tx_in_place and getattr(self, "_described", False):
            flags |= capi.F_REUSE_DESC
        key = ("s", fixed)
        a = self._args.get(key)
        if a is not None:
            a.hdr_templates = templates.data_ptr() if templates is not None else None
            a.req_token = tokens.data_ptr() if tokens is not None else None
        if a is None:
            sizes = self.w.resp_sizes
            fx = int(sizes[0]) if fixed and len(sizes) and bool((sizes == sizes[0]).all()) else 0
            a = ctx.scatter_args(self.rx, self.tx, self.tx_slot, self.hdr_src_slot, self.resp_first,
                                 None if fx else self.resp_size, fx, self.n_req, self.n_frames,
                                 self.w.mtu, self.resp_app, self.resp_offsets, 0, templates, tokens)
            self._args[key] = a
        a.flags = self.w.flags | flags
        return a

    def scatter(self, ctx: SgContext, flags: int = 0, fixed: bool = True, fuse: bool = True,
                templates: Optional[torch.Tensor] = None, tokens: Optional[torch.Tensor] = None,
                reuse: bool = False) -> None:
        ctx.scatter_batch_raw(self.scatter_call(ctx, flags, fixed, fuse, templates, tokens, reuse))

    def shunt(self, ctx: SgContext, flags: int = 0, rule: bool = True) -> None:
        """Gather and scatter of this workload as one pass of the shunter's
        loop (one launch where the two calls can share one)."""
        g = self.gather_call(ctx, flags, rule=rule)
        s = self.scatter_call(ctx, flags, fuse=rule)
        ctx.shunt_batch_raw(g, s)
