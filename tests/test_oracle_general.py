"""Pins for the oracle's general (data-dependent fan-out) branch and the seam's entry helper.

Each function is checked against something it must reduce to -- a library routine on inputs where
that routine is unambiguous (``torch.nonzero``, ``torch.topk`` over distinct keys, ``scatter_add``
of distinct powers of two, stable ``torch.sort``), pure-Python brute force on small inputs, or the
quota branch it has to agree with on an equal-quota routing.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import equal_quota_routing
from oracle import terrace_oracle as orc


def _free_routing(T, k, E, seed):
    rng = np.random.default_rng(seed)
    return np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int64)


GEOMS = [(4, 2, 8, 9, 3), (32, 8, 64, 40, 4), (16, 8, 32, 17, 5), (64, 8, 128, 33, 6), (8, 4, 8, 1, 2)]


@pytest.mark.parametrize("world,rpn,E,T,k", GEOMS)
def test_build_expansion_is_the_sum_of_distinct_powers_of_two(world, rpn, E, T, k):
    e = _free_routing(T, k, E, 7)
    slots = (E // world) * rpn
    u_src, u_node, counts, inverse = orc.plan_ta2a(e, world, E, rpn)
    mask = orc.build_expansion(e, inverse, u_src.size, world, E, rpn)
    # library form, as the reference writes it: scatter_add of 2**slot per (token, expert)
    lib = torch.zeros(u_src.size, dtype=torch.int64)
    lib.scatter_add_(0, torch.from_numpy(inverse), torch.from_numpy(np.int64(1) << (e.reshape(-1) % slots)))
    assert np.array_equal(mask, lib.numpy())
    # by definition: bit j of row (n, t) <=> expert n*slots + j is one of t's
    for r in range(u_src.size):
        want = sum(1 << int(x % slots) for x in e[u_src[r]] if x // slots == u_node[r])
        assert int(mask[r]) == want
    assert np.array_equal(np.array([bin(int(m)).count("1") for m in mask]).sum(), T * k)


def test_build_expansion_refuses_more_than_63_slots():
    e = _free_routing(4, 2, 128, 1)
    with pytest.raises(ValueError, match="exceeds the int64 mask"):
        orc.build_expansion(e, np.zeros(8, np.int64), 4, 2, 128, 2)


def test_sparse_gate_plane_by_definition():
    world, rpn, E, T, k = 32, 8, 64, 21, 4
    e = _free_routing(T, k, E, 3)
    slots = (E // world) * rpn
    gates = np.random.default_rng(4).standard_normal((T, k)).astype(np.float32)
    u_src, u_node, _, inverse = orc.plan_ta2a(e, world, E, rpn)
    plane = orc.sparse_gate_plane(e, gates, inverse, u_src.size, slots)
    want = np.zeros_like(plane)
    for t in range(T):
        for j in range(k):
            r = [i for i in range(u_src.size) if u_src[i] == t and u_node[i] == e[t, j] // slots]
            assert len(r) == 1
            want[r[0], e[t, j] % slots] = gates[t, j]
    assert np.array_equal(plane, want)
    assert np.count_nonzero(plane) == T * k


@pytest.mark.parametrize("slots", [1, 5, 16, 24, 25, 40, 63])
def test_expand_arrival_general_is_nonzero_order(slots):
    rng = np.random.default_rng(slots)
    rmask = rng.integers(0, 1 << slots, size=37, dtype=np.int64)
    rmask[3] = 0
    r, c = orc.expand_arrival(rmask, slots, None)
    bits = torch.tensor([[(int(m) >> j) & 1 for j in range(slots)] for m in rmask])
    lr, lc = torch.nonzero(bits, as_tuple=True)
    assert np.array_equal(r, lr.numpy()) and np.array_equal(c, lc.numpy())


@pytest.mark.parametrize("slots,quota", [(8, 2), (16, 4), (24, 3), (32, 2), (63, 5), (4, 4)])
def test_expand_arrival_quota_is_topk_over_the_distinct_key(slots, quota):
    rng = np.random.default_rng(slots * 10 + quota)
    rows = []
    for i in range(50):
        n_set = quota if i % 5 else rng.integers(0, quota + 1)        # some rows hold fewer than quota
        cols = rng.permutation(slots)[:n_set]
        rows.append(sum(1 << int(c) for c in cols))
    rmask = np.array(rows, dtype=np.int64)
    r, c = orc.expand_arrival(rmask, slots, quota)
    bits = torch.tensor([[(int(m) >> j) & 1 for j in range(slots)] for m in rmask], dtype=torch.float32)
    key = bits * slots + (slots - 1 - torch.arange(slots, dtype=torch.float32))     # distinct per row
    lib = torch.topk(key, quota, dim=1).indices
    assert np.array_equal(c, lib.reshape(-1).numpy())
    assert np.array_equal(r, np.repeat(np.arange(50), quota))
    full = [i for i in range(50) if bin(int(rmask[i])).count("1") == quota]
    for i in full:                                  # a full row: exactly its set columns, ascending
        assert [int(x) for x in c[i * quota:(i + 1) * quota]] == [j for j in range(slots) if (int(rmask[i]) >> j) & 1]


def test_general_branch_reproduces_the_quota_branch_on_equal_quota_routing(literals):
    """The reference's claim for its quota wire format (terrace/ta2a_fwd.py:184-203): the slot
    table holds, row by row, exactly the pairs the bitmask branch extracts, in the same order --
    so the arrival chain of either branch sees one pair sequence."""
    for world, rpn, E, T, k, M in literals["k2_geometries"]["rows"]:
        slots, q, epr = (E // world) * rpn, k // M, E // world
        if slots > 63:
            continue
        e = equal_quota_routing(T, k, E, world // rpn, M, 5)
        rng = np.random.default_rng(6)
        hidden = rng.standard_normal((T, 8)).astype(np.float32)
        gates = rng.standard_normal((T, k)).astype(np.float32)
        payload, slot_tab, gate_tab, u_src, counts = orc.k2_pack(hidden, e, gates, world, E, rpn, M)
        _, _, _, inverse = orc.plan_ta2a(e, world, E, rpn)
        mask = orc.build_expansion(e, inverse, T * M, world, E, rpn)
        for quota in (None, q):
            r, c = orc.expand_arrival(mask, slots, quota)
            assert np.array_equal(r, np.repeat(np.arange(T * M), q))
            assert np.array_equal(c, slot_tab.reshape(-1))
        plane = orc.sparse_gate_plane(e, gates, inverse, T * M, slots)
        gen = orc.arrival_pairs(payload, r, c, plane, epr, rpn)
        quo = orc.k1_arrival(payload, slot_tab, gate_tab, q, epr, rpn)
        for a, b in zip(gen[:5], quo):
            assert np.array_equal(a, b)


def test_arrival_pairs_is_a_stable_library_sort():
    rng = np.random.default_rng(11)
    R, slots, epr, rpn, H = 30, 12, 3, 4, 5
    rmask = rng.integers(0, 1 << slots, size=R, dtype=np.int64)
    r, c = orc.expand_arrival(rmask, slots, None)
    rx = rng.standard_normal((R, H)).astype(np.float32)
    rgate = rng.standard_normal((R, slots)).astype(np.float32)
    send, gp, r2, s2, i_send, ordo = orc.arrival_pairs(rx, r, c, rgate, epr, rpn)
    lib = torch.sort(torch.from_numpy(c // epr), stable=True).indices.numpy()
    assert np.array_equal(ordo, lib)
    assert np.array_equal(r2, r[lib]) and np.array_equal(s2, c[lib])
    assert np.array_equal(send, rx[r[lib]]) and np.array_equal(gp, rgate[r[lib], c[lib]])
    assert np.array_equal(i_send, np.bincount(c // epr, minlength=rpn))
    assert np.all(np.diff(s2 // epr) >= 0)


def test_routing_map_to_topk_is_nonzero_plus_gather_and_fails_loud():
    rng = np.random.default_rng(2)
    T, E, k = 19, 24, 5
    e = np.sort(np.stack([rng.permutation(E)[:k] for _ in range(T)]), 1)
    rm = np.zeros((T, E), dtype=bool)
    rm[np.arange(T)[:, None], e] = True
    probs = rng.random((T, E)).astype(np.float32)
    got_e, got_g = orc.routing_map_to_topk(rm, probs)
    assert np.array_equal(got_e, e)
    assert np.array_equal(got_g, torch.from_numpy(probs).gather(1, torch.from_numpy(e)).numpy())
    assert np.array_equal(got_e.reshape(-1), torch.nonzero(torch.from_numpy(rm))[:, 1].numpy())
    bad = rm.copy()
    bad[3, e[3, 0]] = False
    with pytest.raises(RuntimeError, match="exactly k experts"):
        orc.routing_map_to_topk(bad, probs)
    with pytest.raises(RuntimeError, match="all-empty"):
        orc.routing_map_to_topk(np.zeros((4, 8), bool), np.zeros((4, 8), np.float32))


def test_pair_places_by_definition(literals):
    """where[t, j] is the one place of the expert-order buffer holding token t's copy for expert
    expert_idx[t, j]: checked by walking the chain backwards from every place."""
    for world, rpn, E, T, k, M in literals["k2_geometries"]["rows"]:
        slots, q, epr = (E // world) * rpn, k // M, E // world
        e = equal_quota_routing(T, k, E, world // rpn, M, 9)
        rng = np.random.default_rng(3)
        hidden = rng.standard_normal((T, 4)).astype(np.float32)
        gates = rng.standard_normal((T, k)).astype(np.float32)
        payload, slot_tab, gate_tab, u_src, counts = orc.k2_pack(hidden, e, gates, world, E, rpn, M)
        _, u_node, _, _ = orc.plan_ta2a(e, world, E, rpn)
        send, gp, r_idx, slot_idx, _ = orc.k1_arrival(payload, slot_tab, gate_tab, q, epr, rpn)
        permuted, order, tpe = orc.regroup(send, slot_idx, slots)
        where, tok = orc.pair_places(order, r_idx, slot_idx, u_src, u_node, e, slots)
        assert np.array_equal(np.sort(where.reshape(-1)), np.arange(T * k))          # a bijection onto the places
        assert np.array_equal(permuted, hidden[tok])                                 # the place holds that token's row
        for t in range(T):
            for j in range(k):
                i = where[t, j]
                assert tok[i] == t
                assert gp[order][i] == gates[t, j]                                   # and that expert's gate
                # local expert of the place = node-local slot of expert (t, j)
                assert np.searchsorted(np.cumsum(tpe), i, side="right") == e[t, j] % slots
