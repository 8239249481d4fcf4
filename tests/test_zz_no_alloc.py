"""The entry point that allocates nothing (terrace_k1_arrival_static) against the CPU oracle's arrival chain and
against terrace_k1_arrival, through the C ABI: same planes and rows bit for bit, on calls in a row that share the
library's fixed scratch array -- the second on a smaller input, so anything the first left behind would show --
and captured in a HIP graph after terrace_static_init(), replayed between eager calls."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from conftest import arrival_plane
from oracle import terrace_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _planes(R, H, quota, epr, rpn, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    rx = torch.randn((R, H), generator=g).to(dtype).to(DEV)
    rslot = torch.from_numpy(arrival_plane(R, quota, epr, rpn, seed)).to(DEV)
    rgate = torch.rand((R, quota), generator=g).to(dtype).to(DEV)
    return rx, rslot, rgate


def _outputs(R, H, quota, rpn, dtype):
    P = R * quota
    i64 = dict(dtype=torch.int64, device=DEV)
    return (torch.empty((P, H), dtype=dtype, device=DEV), torch.empty((P,), dtype=dtype, device=DEV),
            torch.empty((P,), **i64), torch.empty((P,), **i64), torch.empty((rpn,), **i64), torch.empty((P,), **i64),
            torch.empty((4,), dtype=torch.int32, device=DEV))


def test_static_scratch_entry_point_matches_the_workspace_one():
    import terrace.ops as tops
    from terrace import _hip
    tops.reset()
    assert tops.status().loaded, tops.status().reason
    cases = [(20000, 512, 2, 4, 8, torch.bfloat16, 11),      # 40000 pairs, several units per bucket
             (777, 96, 4, 2, 8, torch.float32, 12),          # smaller: would read stale scratch if any were trusted
             (0, 64, 2, 4, 8, torch.bfloat16, 13)]           # empty arrival
    for R, H, quota, epr, rpn, dtype, seed in cases:
        print("[case] k1_arrival_static", R, H, quota, epr, rpn, dtype, flush=True)
        rx, rslot, rgate = _planes(R, H, quota, epr, rpn, dtype, seed)
        want = tops.k1_arrival_raw(rx, rslot, rgate, quota, epr, rpn, 0, want_pair_pos=True)
        out = _outputs(R, H, quota, rpn, dtype)
        before = torch.cuda.memory_allocated()
        tops.k1_arrival_static(rx, rslot, rgate, quota, epr, rpn, 0, out)
        assert torch.cuda.memory_allocated() == before          # the binding itself made no tensor
        torch.cuda.synchronize()
        names = ("send_buf", "gate_pairs", "r_idx", "slot_idx", "i_send", "pair_pos")
        for name, got, ref in zip(names, out, want):
            assert got.dtype == ref.dtype and got.shape == ref.shape, name
            assert torch.equal(got.view(torch.uint8) if got.is_floating_point() else got,
                               ref.view(torch.uint8) if ref.is_floating_point() else ref), f"{name} differs (R={R})"
        # and against the oracle's arrival chain (rows and gates as raw bits)
        bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
        o = orc.k1_arrival(rx.view(bits).cpu().numpy(), rslot.cpu().numpy(), rgate.view(bits).cpu().numpy(), quota, epr,
                           rpn)
        for name, got, ref in zip(names[:5], out, o):
            got = got.view(bits) if got.is_floating_point() else got
            assert np.array_equal(got.cpu().numpy(), ref), f"{name} differs from the oracle (R={R})"
        assert np.array_equal(out[5].cpu().numpy(), orc.arrival_positions(rslot.cpu().numpy(), epr, rpn).reshape(-1))
        if R:
            assert int(out[6][0]) == 0


def test_static_scratch_entry_point_in_a_hip_graph():
    """After terrace_static_init() the call is kernel launches only, so a stream capture can record it.  Every
    replay -- with eager calls on other inputs between them, which overwrite the shared scratch -- must reproduce
    the workspace entry point's result for whatever the captured input tensors hold at that time."""
    import terrace.ops as tops
    from terrace import _hip
    assert _hip.load().terrace_static_init() == 0
    assert _hip.load().terrace_static_init() == 0           # idempotent
    R, H, quota, epr, rpn, dtype = 3000, 256, 2, 4, 8, torch.bfloat16
    rx, rslot, rgate = _planes(R, H, quota, epr, rpn, dtype, 21)
    out = _outputs(R, H, quota, rpn, dtype)
    other = _planes(500, 64, 4, 2, 8, torch.float32, 22)
    other_out = _outputs(500, 64, 4, 8, torch.float32)
    tops.k1_arrival_static(rx, rslot, rgate, quota, epr, rpn, 0, out)        # eager warm-up of every kernel
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            tops.k1_arrival_static(rx, rslot, rgate, quota, epr, rpn, 0, out)
    torch.cuda.current_stream().wait_stream(side)
    names = ("send_buf", "gate_pairs", "r_idx", "slot_idx", "i_send", "pair_pos")
    for rep in range(3):
        print("[case] k1_arrival_static graph replay", rep, flush=True)
        # new contents in the captured input tensors, and an eager call that dirties the scratch
        fresh = _planes(R, H, quota, epr, rpn, dtype, 30 + rep)
        for dst, src in zip((rx, rslot, rgate), fresh):
            dst.copy_(src)
        tops.k1_arrival_static(*other, 4, 2, 8, 0, other_out)
        for t in out:
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = tops.k1_arrival_raw(rx, rslot, rgate, quota, epr, rpn, 0, want_pair_pos=True)
        for name, got, ref in zip(names, out, want):
            assert torch.equal(got.view(torch.uint8) if got.is_floating_point() else got,
                               ref.view(torch.uint8) if ref.is_floating_point() else ref), f"{name} (replay {rep})"


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from terrace import _hip
    lib = _hip.load()
    cap = _hip.query("terrace_static_scratch_bytes")
    assert cap == 4 << 20
    R = 2_000_000                                   # 4M pairs: the position plane alone is 16 MB
    assert _hip.query("terrace_k1_arrival_workspace", R, 2, 8) > cap
    rc = lib.terrace_k1_arrival_static(None, None, None, R, 0, 2, 2, 4, 8, 0, None, None, None, None, None, None,
                                       None, None)
    assert rc == _hip.E2BIG
    assert b"scratch" in lib.terrace_strerror(rc)
