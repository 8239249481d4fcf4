"""The one-pass Hop-B local scatter (terrace_hopb_scatter) against the CPU oracle's composition of the arrival
chain and the expert-order regroup, bit for bit, through the C ABI -- and against the two-step operators it
replaces on the device."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import arrival_plane
from oracle import terrace_oracle as orc
from test_gpu_parity import DEV, DT, announce, same, to_np

pytestmark = pytest.mark.gpu


def _check(R, H, quota, epr, rpn, fmt, capacity, seed, first_slot=0, degenerate=False, gates=True):
    import terrace.ops as tops
    n_local = epr * rpn
    g = torch.Generator().manual_seed(seed)
    rx = torch.randn((R, H), generator=g).to(DT[fmt])
    rslot = arrival_plane(R, quota, epr, rpn, seed, degenerate) + first_slot
    rgate = torch.rand((R, quota), generator=g).to(DT[fmt])
    out = tops.hopb_scatter(rx.to(DEV), torch.from_numpy(rslot).to(DEV), rgate.to(DEV) if gates else None, quota,
                            n_local, first_slot, capacity, want_pairs=True)
    permuted, place, kept, counts, kept_per, pgate, pairs = orc.hopb_local_scatter(
        to_np(rx), rslot, to_np(rgate), quota, n_local, first_slot, capacity)
    same(out["permuted"], permuted, "permuted"), same(out["place"], place, "place")
    same(out["tokens_per_expert"], counts, "tokens_per_expert"), same(out["kept_per_expert"], kept_per, "kept_per_expert")
    same(out["pair_of_place"], pairs, "pair_of_place")
    if capacity is None:
        assert out["kept"] is None
    else:
        same(out["kept"], kept, "kept")
    if gates:
        same(out["permuted_gate"], pgate, "permuted_gate")
    else:
        assert out["permuted_gate"] is None
    if R:
        assert out["status"].tolist()[0] == 0
    return out


@pytest.mark.parametrize("fmt", ["f32", "bf16"])
@pytest.mark.parametrize("capacity", [None, 7, 1 << 20])
def test_hopb_scatter_on_the_reference_arrival_geometries(literals, fmt, capacity):
    for R, quota, epr, rpn, H in literals["k1_geometries"]["rows"]:
        announce("hopb", R, H, quota, epr, rpn, fmt, capacity)
        _check(R, H, quota, epr, rpn, fmt, capacity, seed=R + H + quota)


@pytest.mark.parametrize("R,H,quota,epr,rpn,fmt,capacity", [
    (0, 64, 2, 4, 8, "bf16", None), (0, 64, 2, 4, 8, "bf16", 5), (1, 8, 1, 1, 1, "f32", None),
    (300, 1000, 3, 2, 8, "f32", 40), (5000, 512, 2, 4, 8, "bf16", 300), (9000, 3696, 2, 4, 8, "f16", None),
    (70000, 64, 2, 4, 8, "bf16", 4000), (2500, 6, 4, 1, 8, "f32", 0), (4100, 13, 2, 3, 5, "f32", 600),
    (64, 7168, 2, 4, 8, "bf16", None), (200, 24, 6, 32, 8, "f32", 4),
])
def test_hopb_scatter_sizes_widths_and_capacities(R, H, quota, epr, rpn, fmt, capacity):
    announce("hopb sizes", R, H, quota, epr, rpn, fmt, capacity)
    _check(R, H, quota, epr, rpn, fmt, capacity, seed=R + H)
    _check(R, H, quota, epr, rpn, fmt, capacity, seed=R + H + 1, first_slot=9, gates=False)


def test_hopb_scatter_degenerate_rows_overflow_one_expert():
    announce("hopb degenerate")
    out = _check(500, 32, 2, 4, 8, "f32", 64, seed=3, degenerate=True)          # every pair names slot 0
    assert out["tokens_per_expert"].tolist()[0] == 1000 and out["kept_per_expert"].tolist()[0] == 64
    assert int(out["kept"].sum()) == 64


@pytest.mark.parametrize("capacity", [None, 50])
def test_hopb_scatter_equals_the_two_step_operators_on_the_device(capacity):
    import terrace.ops as tops
    from terrace.ta2a_fwd import _regroup_with_place
    announce("hopb vs two-step", capacity)
    R, H, quota, epr, rpn = 3000, 256, 2, 4, 8
    g = torch.Generator().manual_seed(5)
    rx = torch.randn((R, H), generator=g).to(torch.bfloat16).to(DEV)
    rslot = torch.from_numpy(arrival_plane(R, quota, epr, rpn, 5)).to(DEV)
    rgate = torch.rand((R, quota), generator=g).to(torch.bfloat16).to(DEV)
    send_buf, gate_pairs, r_idx, slot_idx, i_send, pair_pos = tops.k1_arrival_raw(rx, rslot, rgate, quota, epr, rpn, 0,
                                                                                  want_pair_pos=True)
    if capacity is None:
        permuted, order, tpe, place = _regroup_with_place(send_buf, slot_idx, epr * rpn)
    else:
        permuted, place, kept, tpe, kpe = tops.regroup(send_buf, slot_idx, epr * rpn, 0, capacity)
    ws = []
    first = tops.hopb_scatter(None, rslot, rgate, quota, epr * rpn, 0, capacity, workspace_out=ws)
    assert first["permuted"] is None
    moved = tops.hopb_scatter_move(rx, ws[0], quota, epr * rpn, capacity)
    one = tops.hopb_scatter(rx, rslot, rgate, quota, epr * rpn, 0, capacity)
    assert torch.equal(one["permuted"], permuted) and torch.equal(moved, permuted)
    assert torch.equal(one["place"], place[pair_pos]) and torch.equal(first["place"], one["place"])
    assert torch.equal(one["tokens_per_expert"], tpe)
    if capacity is not None:
        assert torch.equal(one["kept"], kept[pair_pos]) and torch.equal(one["kept_per_expert"], kpe)


def test_hopb_scatter_refuses_bad_arguments_and_contains_bad_ids():
    import terrace.ops as tops
    from terrace import _hip
    announce("hopb bad arguments")
    lib = _hip.load()
    s = _hip.stream(DEV)
    i64 = torch.zeros(64, dtype=torch.int64, device=DEV)
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    st = torch.zeros(4, dtype=torch.int32, device=DEV)
    args = lambda R, quota, n_local, cap, ws_bytes: (None, _hip.ptr(i64), None, R, 0, 4, quota, 0, n_local, cap, None,
                                                     None, _hip.ptr(i64), None, None, _hip.ptr(i64), None, None, None, 0,
                                                     _hip.ptr(st), _hip.ptr(ws), ws_bytes, s)
    assert lib.terrace_hopb_scatter(*args(16, 2, 0, -1, ws.numel())) == _hip.EINVAL
    assert lib.terrace_hopb_scatter(*args(16, 0, 8, -1, ws.numel())) == _hip.EINVAL
    assert lib.terrace_hopb_scatter(*args(16, 2, 8, -1, 16)) == _hip.ENOSPC
    assert lib.terrace_hopb_scatter(*args(1 << 40, 2, 8, -1, ws.numel())) == _hip.EINVAL
    assert lib.terrace_hopb_scatter_move(None, 16, 64, 2, 8, -1, _hip.ptr(ws), _hip.ptr(ws), 16, s) == _hip.EINVAL
    assert lib.terrace_hopb_scatter_move(None, 0, 64, 2, 8, -1, None, None, 0, s) == _hip.OK
    # slot ids outside [first_slot, first_slot + n_local) are contained and reported, never used as an address
    rslot = torch.tensor([[0, 3], [40, 2], [-5, 1]], device=DEV)
    rx = torch.arange(3 * 4, dtype=torch.float32, device=DEV).view(3, 4)
    out = tops.hopb_scatter(rx, rslot, None, 2, 4, 0, None)
    torch.cuda.synchronize()
    assert out["status"].tolist()[0] & _hip.FAULT_ID_RANGE
    assert bool(((out["place"] >= 0) & (out["place"] < 6)).all()) and int(out["tokens_per_expert"].sum()) == 6
