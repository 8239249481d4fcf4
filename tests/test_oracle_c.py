"""Pins the C restatement (the multi-core CPU baseline) bit for bit to the numpy oracle."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import arrival_plane, equal_quota_routing
from oracle import c_oracle as corc
from oracle import terrace_oracle as orc

pytestmark = pytest.mark.skipif(not corc.available(), reason="oracle/_c/libterrace_oracle.so not built "
                                                             "(python oracle/build_c.py)")


@pytest.mark.parametrize("T,E,Ng,k,M", [(300, 64, 8, 8, 4), (257, 256, 8, 8, 4), (100, 128, 16, 8, 2), (50, 24, 3, 6, 3),
                                        (64, 8, 8, 2, 2)])
def test_route(T, E, Ng, k, M):
    rng = np.random.default_rng(T)
    aff = rng.standard_normal((T, E)).astype(np.float32)
    aff[3] = 0.5                                         # ties
    bias = (rng.standard_normal(E) * 0.1).astype(np.float32)
    ga = np.exp(aff - aff.max(-1, keepdims=True)).astype(np.float32)
    for pool in (1, 2):
        for gate_aff in (None, ga):
            a = corc.t_route(aff, bias, E, Ng, k, M, pool, gate_aff)
            b = orc.t_route(aff, bias, E, Ng, k, M, pool, gate_affinity=gate_aff)
            for x, y in zip(a, b):
                assert x.dtype == y.dtype and np.array_equal(x, y)


def test_k2_pack(literals):
    for world, rpn, E, T, k, M in literals["k2_geometries"]["rows"]:
        rng = np.random.default_rng(T + k)
        e = equal_quota_routing(T, k, E, world // rpn, M, 500)
        for dt in (np.float32, np.uint16):
            hidden = rng.integers(0, 60000, (T, 16)).astype(dt)
            gates = rng.integers(0, 60000, (T, k)).astype(dt)
            got = corc.k2_pack(hidden, e, gates, world, E, rpn, M)
            want = orc.k2_pack(hidden, e, gates, world, E, rpn, M)
            for a, b in zip(got[:5], want):
                assert a.dtype == b.dtype and np.array_equal(a, b)
            _, u_node, _, inverse = orc.plan_ta2a(e, world, E, rpn, M)
            pair_tab, order = orc.token_pair_table(e, inverse, k // M)
            assert np.array_equal(got[5]["u_node"], u_node) and np.array_equal(got[5]["inverse"], inverse)
            assert np.array_equal(got[5]["pair_table"], pair_tab) and np.array_equal(got[5]["sort_order"], order)
    with pytest.raises(ValueError):
        corc.k2_pack(np.zeros((4, 4), np.float32), np.array([[0, 2, 3, 5]] * 4), np.zeros((4, 4), np.float32), 4, 8, 2, 2)


def test_k1_and_regroup(literals):
    for R, q, epr, rpn, H in literals["k1_geometries"]["rows"]:
        rslot = arrival_plane(R, q, epr, rpn, 100)
        rng = np.random.default_rng(R)
        rx = rng.integers(0, 60000, (R, H)).astype(np.uint16)
        rgate = rng.integers(0, 60000, (R, q)).astype(np.uint16)
        got = corc.k1_arrival(rx, rslot, rgate, q, epr, rpn)
        want = orc.k1_arrival(rx, rslot, rgate, q, epr, rpn)
        for a, b in zip(got[:5], want):
            assert a.dtype == b.dtype and np.array_equal(a, b)
        assert np.array_equal(got[5], orc.arrival_positions(rslot, epr, rpn))
        slots = epr * rpn
        perm, order, tpe = orc.regroup(want[0], want[3], slots)
        cp, place, kept, ctpe = corc.regroup(want[0], want[3], slots)
        assert np.array_equal(cp, perm) and np.array_equal(ctpe, tpe) and np.array_equal(np.argsort(place), order)
        cap = max(1, (R * q) // slots)
        wp, wdest, wkept, wt, _ = orc.regroup(want[0], want[3], slots, capacity=cap)
        cp, place, kept, ctpe = corc.regroup(want[0], want[3], slots, capacity=cap)
        assert np.array_equal(cp, wp) and np.array_equal(place, wdest) and np.array_equal(kept, wkept)


@pytest.mark.parametrize("in_fmt,out_fmt", [("f32", "f32"), ("bf16", "bf16"), ("bf16", "f32"), ("fp8", "bf16")])
def test_combine(in_fmt, out_fmt):
    rng = np.random.default_rng(5)
    H = 256
    x = rng.standard_normal((40, H)).astype(np.float32)
    src = {"f32": x, "bf16": orc.f32_to_bf16(x), "fp8": orc.fp8_quantise_rows(x)}[in_fmt]
    idx = rng.integers(-1, 40, (17, 5))
    w = rng.random((17, 5)).astype(np.float32)
    for weights in (w, None):
        a = corc.combine(src, idx, weights, in_fmt, out_fmt, hidden=H)
        b = orc.combine(src, idx, weights, in_fmt, out_fmt, hidden=H)
        assert a.dtype == b.dtype and np.array_equal(a, b)
    assert corc.threads() >= 1
