"""The torch-CPU operator chain that serves as the benchmark's CPU baseline, held to the numpy oracle plane by
plane: it must compute the same path, or timing it says nothing."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import terrace_oracle as orc
from oracle import torch_chain as tch


@pytest.mark.parametrize("T,E,Ng,k,M,rpn,H,capacity", [(257, 64, 8, 4, 2, 8, 24, None), (300, 256, 8, 8, 4, 8, 16, 12),
                                                       (64, 128, 16, 8, 2, 8, 8, None)])
def test_torch_chain_equals_the_oracle(T, E, Ng, k, M, rpn, H, capacity):
    g = torch.Generator().manual_seed(T + E)
    logits = torch.randn(T, E, generator=g)
    bias = torch.randn(E, generator=g) * 0.1
    x = torch.randn(T, H, generator=g)
    world = Ng * rpn
    epr, slots, q = E // world, (E // world) * rpn, k // M
    e, gates, grp = tch.t_route(logits, bias, E, Ng, k, M)
    oe, og, ogrp = orc.t_route(logits.numpy(), bias.numpy(), E, Ng, k, M)
    assert np.array_equal(e.numpy(), oe) and np.array_equal(grp.numpy(), ogrp)
    assert np.allclose(gates.numpy(), og, rtol=1e-5, atol=0)
    gates = torch.from_numpy(og)
    payload, mask, gate_rows, u_src, counts, inverse = tch.k2_pack(x, e, gates, world, E, rpn, M)
    o = orc.k2_pack(x.numpy(), oe, og, world, E, rpn, M)
    for got, want in zip((payload, mask, gate_rows, u_src, counts), o):
        assert np.array_equal(got.numpy(), want)
    send, gp, r_idx, s_idx, i_send, ordo = tch.k1_arrival(payload, mask, gate_rows, q, epr, rpn)
    oa = orc.k1_arrival(o[0], o[1], o[2], q, epr, rpn)
    for got, want in zip((send, gp, r_idx, s_idx, i_send), oa):
        assert np.array_equal(got.numpy(), want)
    perm, place, tpe = tch.regroup(send, s_idx, slots, capacity)
    if capacity is None:
        operm, order, otpe = orc.regroup(oa[0], oa[3], slots)
        oplace = np.empty_like(order)
        oplace[order] = np.arange(order.size)
    else:
        operm, oplace, _, otpe, _ = orc.regroup(oa[0], oa[3], slots, capacity=capacity)
        assert (oplace < 0).any(), "the case must drop something"
    assert np.array_equal(perm.numpy(), operm) and np.array_equal(place.numpy(), oplace)
    assert np.array_equal(tpe.numpy(), otpe)
    ye = perm * 0.5
    y = tch.combine_two_level(ye, place, r_idx, gp, u_src, u_src.numel(), T)
    _, _, _, oinv = orc.plan_ta2a(oe, world, E, rpn, M)
    pair_tab, sort_order = orc.token_pair_table(oe, oinv, q)
    pos = orc.arrival_positions(o[1], epr, rpn)
    where = oplace[pos[pair_tab]]
    want = orc.gather_reduce(ye.numpy(), where, np.take_along_axis(og, sort_order, 1))
    assert np.abs(y.numpy() - want).max() <= 1e-5 * max(np.abs(want).max(), 1.0)
