"""HIP batched gather / scatter against the CPU oracle on the five workloads,
bit for bit, through the C ABI."""
import numpy as np
import pytest
import torch

from splitrpc_amd import synth
from splitrpc_amd.engine import DeviceWorkload

from helpers import expected_gather, expected_scatter, first_diff

pytestmark = pytest.mark.gpu

CASES = [(1, None), (2, None), (3, None), (4, None), (5, None), (2, 1), (4, 7), (5, 2)]


MODES = {
    # request offsets by prefix scan, descriptor pass for gather and scatter
    "scan": dict(fixed=False, rule=False, fuse=False),
    # one declared size: offsets are multiples, descriptor pass still runs
    "fixed": dict(fixed=True, rule=False, fuse=False),
    # one declared size + fragmenting rule: copy kernels derive the descriptors
    "rule": dict(fixed=True, rule=True, fuse=True),
}


# the reference's own 64-byte p2p_rpc_hdr (src/p2p_rpc.h:10-17; lengths from a table, as from the
# NIC) at the full size of the configurations the benchmark runs it on
REF64_CASES = [(2, None), (1, None), (5, None), (3, None)]


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("cfg,n_req", REF64_CASES)
def test_gather_scatter_bit_exact_with_the_reference_header(ctx, cfg, n_req, mode):
    test_gather_scatter_bit_exact(ctx, cfg, n_req, mode, profile=synth.HDR_REF64)


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("cfg,n_req", CASES)
def test_gather_scatter_bit_exact(ctx, cfg, n_req, mode, profile=synth.HDR_BL58):
    fixed, rule, fuse = MODES[mode]["fixed"], MODES[mode]["rule"], MODES[mode]["fuse"]
    w = synth.make_workload(cfg, n_req, profile=profile)
    print(f"case cfg={cfg} n_req={w.n_req} frags={w.n_frags} frames={w.n_resp_frames} mode={mode} profile={profile}",
          flush=True)
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    ctx.set_cursor(1, 0)

    dw.gather(ctx, fixed=fixed, rule=rule)
    if w.in_tensor_sizes:
        exp, _, _ = expected_gather(w)
        for t, e in zip(dw.in_tensors, exp):
            got = t.cpu().numpy()
            assert np.array_equal(got, e), first_diff(got, e)
        gathered = None
    else:
        exp, offs, cur = expected_gather(w, arena_cap=dw.req_app.cap)
        got = dw.req_arena.cpu().numpy()
        assert np.array_equal(got, exp), first_diff(got, exp)
        assert np.array_equal(dw.req_offsets.cpu().numpy().view(np.uint64), offs)
        assert ctx.get_cursor(0) == cur
        gathered = exp

    dw.scatter(ctx, fixed=fixed, fuse=fuse)
    exp_tx, offs, cur = expected_scatter(w, gathered, resp_cap=dw.resp_app.cap if not w.out_tensor_sizes else None)
    got_tx = dw.tx_ring.cpu().numpy()
    assert np.array_equal(got_tx, exp_tx), first_diff(got_tx, exp_tx)
    if dw.resp_offsets is not None:
        assert np.array_equal(dw.resp_offsets.cpu().numpy().view(np.uint64), offs)
        assert ctx.get_cursor(1) == cur


def test_gather_with_explicit_lengths(ctx):
    w = synth.make_workload(2, 2)
    dw = DeviceWorkload(w)
    ctx.set_cursor(0, 0)
    dw.gather(ctx, use_frag_len=True)
    exp, _, _ = expected_gather(w, arena_cap=dw.req_app.cap)
    assert np.array_equal(dw.req_arena.cpu().numpy(), exp)
