"""sg_hip_pack_tables: fragment tables kept in pinned host memory (one per
request, 32-bit offsets from a packet base, as the receive thread files them)
pulled by the device into the CSR tables of the batched calls.  The pulled
tables are held against the tables the generator made, and a gather over them
against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest
import torch

from splitrpc_amd import capi, synth
from splitrpc_amd.engine import DeviceWorkload, SgContext

from helpers import expected_gather, first_diff

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tables_of(w, dw, pkt_base, order, n_tables):
    """Host image of `n_tables` fragment tables; request r keeps table order[r]."""
    hl = 64 if w.profile else 58
    t = np.full((n_tables, 2, capi.MAX_BI_SIZE), 0xFFFFFFFF, np.uint32)
    ring = dw.ring.data_ptr()
    for r in range(w.n_req):
        f0, f1 = int(w.req_first[r]), int(w.req_first[r + 1])
        addr = ring + w.frag_slot[f0:f1].astype(np.int64) * w.slot_size + hl
        t[order[r], 0, :f1 - f0] = ((addr - pkt_base) >> 1).astype(np.uint32)
        t[order[r], 1, :f1 - f0] = w.frag_len[f0:f1]
    return t


@pytest.mark.parametrize("where", ["pinned", "device"])
@pytest.mark.parametrize("name,profile", [("lenet", synth.HDR_BL58), ("resnet50", synth.HDR_REF64),
                                          ("ragged", synth.HDR_BL58), ("medium", synth.HDR_BL58)])
def test_pulled_tables_equal_the_tables_a_host_walk_makes(name, profile, where):
    if name == "lenet":
        w = synth.make_workload(1, 40, profile=profile)      # 3 fragments per request: one step of a group's lanes
    elif name == "resnet50":
        w = synth.make_workload(2, 3, profile=profile)       # 431 fragments: seven steps of sixteen lanes
    elif name == "medium":
        w = synth.make_custom([1400 * 40 + 7] * 9, [64] * 9, seed=81, profile=profile)  # 41: one step
    else:
        rng = np.random.default_rng(8)
        w = synth.make_custom([int(x) for x in rng.integers(0, 60000, 37)], [64] * 37, seed=82, profile=profile)
    print(f"case pack {name} {where} n_req={w.n_req} frags={w.n_frags}", flush=True)
    ctx = SgContext(0)
    dw = DeviceWorkload(w)
    pkt_base = (dw.ring.data_ptr() - 4096) & ~1
    n_tables = w.n_req + 5
    order = np.random.default_rng(3).permutation(n_tables)[:w.n_req]
    img = _tables_of(w, dw, pkt_base, order, n_tables)
    idx = np.ascontiguousarray(order, np.uint32).view(np.int32)
    first = np.ascontiguousarray(w.req_first, np.uint32).view(np.int32)
    blob = np.arange(1000, dtype=np.int32)
    if where == "pinned":
        tables = torch.from_numpy(img.view(np.int32)).pin_memory()
        t_idx, t_first, t_blob = (torch.from_numpy(x.copy()).pin_memory() for x in (idx, first, blob))
    else:
        tables = torch.from_numpy(img.view(np.int32)).to(DEV)
        t_idx, t_first, t_blob = (torch.from_numpy(x.copy()).to(DEV) for x in (idx, first, blob))
    fs = torch.full((w.n_frags + 8,), -7, dtype=torch.int32, device=DEV)
    fl = torch.full((w.n_frags + 8,), -7, dtype=torch.int32, device=DEV)
    rf = torch.full((w.n_req + 1,), -7, dtype=torch.int32, device=DEV)
    bd = torch.zeros(1000, dtype=torch.int32, device=DEV)
    a = capi.PackArgs()
    a.tables = tables.data_ptr()
    a.n_tables = n_tables
    a.n_req = w.n_req
    a.table_idx = t_idx.data_ptr()
    a.req_first = t_first.data_ptr()
    a.n_frags = w.n_frags
    a.pkt_base = pkt_base
    a.ring = dw.rx.desc()
    a.frag_slot = fs.data_ptr()
    a.frag_len = fl.data_ptr()
    a.req_first_out = rf.data_ptr()
    a.blob_src = t_blob.data_ptr()
    a.blob_dst = bd.data_ptr()
    a.blob_words = 1000
    torch.cuda.synchronize()
    assert ctx.lib.sg_hip_pack_tables(ctx.h, C.byref(a)) == capi.SG_OK, ctx.lib.sg_hip_last_error(ctx.h).decode()
    ctx.sync()
    assert np.array_equal(fs.cpu().numpy()[:w.n_frags].view(np.uint32), w.frag_slot.astype(np.uint32))
    assert np.array_equal(fl.cpu().numpy()[:w.n_frags].view(np.uint32), w.frag_len.astype(np.uint32))
    assert bool((fs[w.n_frags:] == -7).all()) and bool((fl[w.n_frags:] == -7).all())
    assert np.array_equal(rf.cpu().numpy().view(np.uint32), w.req_first.astype(np.uint32))
    assert np.array_equal(bd.cpu().numpy(), blob)
    # the gather over the pulled tables
    ctx.set_cursor(0, 0)
    ctx.gather_batch(dw.rx, fs, fl, rf, w.n_req, w.n_frags, dw.req_app, dw.req_offsets)
    exp, eoffs, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    got = dw.req_arena.cpu().numpy()
    assert np.array_equal(got, exp), first_diff(got, exp)
    ctx.close()


def test_entries_that_are_no_payload_start_of_the_ring_are_refused_downstream():
    w = synth.make_custom([4200] * 4, [64] * 4, seed=83)
    ctx = SgContext(0)
    dw = DeviceWorkload(w)
    pkt_base = dw.ring.data_ptr() & ~1
    img = _tables_of(w, dw, pkt_base, np.arange(4), 4)
    good = img.copy()
    img[1, 0, 2] += 1                 # two bytes into the payload: no slot starts there
    img[2, 0, 0] = 0xFFFFFFFF         # never filed
    img[3, 0, 1] = ((dw.ring.data_ptr() + w.n_slots * w.slot_size + 58 - pkt_base) >> 1)  # one slot past the ring
    tables = torch.from_numpy(img.view(np.int32)).pin_memory()
    idx = torch.arange(4, dtype=torch.int32).pin_memory()
    first = torch.from_numpy(np.ascontiguousarray(w.req_first, np.uint32).view(np.int32)).pin_memory()
    fs = torch.zeros(w.n_frags, dtype=torch.int32, device=DEV)
    a = capi.PackArgs()
    a.tables, a.n_tables, a.n_req = tables.data_ptr(), 4, 4
    a.table_idx, a.req_first, a.n_frags = idx.data_ptr(), first.data_ptr(), w.n_frags
    a.pkt_base = pkt_base
    a.ring = dw.rx.desc()
    a.frag_slot = fs.data_ptr()
    torch.cuda.synchronize()
    assert ctx.lib.sg_hip_pack_tables(ctx.h, C.byref(a)) == capi.SG_OK
    ctx.sync()
    got = fs.cpu().numpy().view(np.uint32)
    want = w.frag_slot.astype(np.uint32).copy()
    for r, i in ((1, 2), (2, 0), (3, 1)):
        want[int(w.req_first[r]) + i] = 0xFFFFFFFF
    assert np.array_equal(got, want)
    # a gather over them reports the slots it cannot follow and moves nothing (descriptor pass)
    from splitrpc_amd.engine import SgError
    dw.req_arena.fill_(0xAB)
    with pytest.raises(SgError) as e:
        ctx.gather_batch(dw.rx, fs, None, dw.req_first, w.n_req, w.n_frags, dw.req_app, dw.req_offsets)
    assert e.value.code == capi.SG_E_DATA and "slot" in str(e.value)
    assert bool((dw.req_arena == 0xAB).all())
    # refused by the host: a packet base above the ring, an odd one, missing tables
    a.pkt_base = dw.ring.data_ptr() + 2
    assert ctx.lib.sg_hip_pack_tables(ctx.h, C.byref(a)) == capi.SG_E_INVAL
    a.pkt_base = pkt_base
    a.tables = None
    assert ctx.lib.sg_hip_pack_tables(ctx.h, C.byref(a)) == capi.SG_E_INVAL
    assert good is not None
    ctx.close()
