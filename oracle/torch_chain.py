"""The dispatch/combine path as a chain of torch CPU operators -- the CPU baseline of the benchmark.

TEST INFRASTRUCTURE, NOT PRODUCT (as the rest of ``oracle/``): only ``bench.py``'s ``cpu_baseline`` leg and
the test-suite import it.  It restates, with the library primitives the reference itself composes
(``topk`` / ``gather``; ``scatter_`` + ``cumsum`` + ``searchsorted``; row gathers; a composite-key
``argsort`` + ``scatter_add_``; ``index_add_``), what one rank's path computes, so that timing it on the host
cores answers "what does the reference's own op composition cost on a CPU".  Nothing of the reference is
imported or executed; each function cites the lines whose composition it follows.
``tests/test_oracle_torch_chain.py`` holds it to the numpy oracle plane by plane.

The float32-key workarounds of the reference (sorting and scanning in float32 because its device has no fast
integer sort, terrace/ta2a.py:131-137, terrace/ta2a_fwd.py:324-345) are kept: they are part of the op chain
being priced, and exact below 2**24 like there.
"""
from __future__ import annotations

import torch


def t_route(affinity, bias, n_experts, n_groups, top_k, top_groups, gate_affinity=None):
    """terrace/routing.py:86-95 (mode "full", group_score_pool 2)."""
    T = affinity.shape[0]
    g = n_experts // n_groups
    s = affinity + bias
    sg = s.view(T, n_groups, g)
    score = sg.topk(min(2, g), -1).values.mean(-1)
    group_idx = score.topk(top_groups, -1).indices
    picked = sg.gather(1, group_idx[..., None].expand(-1, -1, g))
    local = picked.topk(top_k // top_groups, -1).indices
    expert_idx = (group_idx[..., None] * g + local).reshape(T, top_k)
    gates = (affinity if gate_affinity is None else gate_affinity).gather(1, expert_idx)
    return expert_idx, gates / gates.sum(-1, keepdim=True), group_idx


def plan(expert_idx, world, n_experts, rpn, groups_m):
    """terrace/ta2a.py:98-275, the groups_m fast path: occupancy scatter, float32 cumsum, searchsorted."""
    T, k = expert_idx.shape
    n_nodes = world // rpn
    slots = (n_experts // world) * rpn
    dest = torch.div(expert_idx, slots, rounding_mode="floor")
    occ = torch.zeros(T, n_nodes, dtype=torch.bool)
    occ.scatter_(1, dest, True)
    node_first = occ.t().reshape(-1)
    row_count = torch.cumsum(node_first.to(torch.float32), 0)
    row_pos = (row_count - 1).to(torch.int64)
    sel = torch.searchsorted(row_count, torch.arange(T * groups_m, dtype=torch.float32), right=True)
    u_node = torch.div(sel, T, rounding_mode="floor")
    u_src = sel % T
    counts = occ.to(torch.float32).sum(0).to(torch.int64)
    inverse = row_pos[(dest * T + torch.arange(T).unsqueeze(1)).reshape(-1)]
    return u_src, u_node, counts, inverse


def pack_quota_wire(expert_idx, gates, inverse, n_rows, slots, quota):
    """terrace/ta2a_fwd.py:226-248: per-row argsort, then one row scatter of a [T*M, quota] view."""
    T, k = expert_idx.shape
    order = torch.argsort(expert_idx.to(torch.float32), dim=1)
    slot_vals = (torch.gather(expert_idx, 1, order) % slots).reshape(-1, quota)
    gate_vals = torch.gather(gates, 1, order).reshape(-1, quota)
    rof = torch.gather(inverse.view(T, k), 1, order[:, ::quota]).reshape(-1)
    slot_tab = torch.zeros(n_rows, quota, dtype=torch.int64)
    slot_tab[rof] = slot_vals
    gate_tab = torch.zeros(n_rows, quota, dtype=gates.dtype)
    gate_tab[rof] = gate_vals
    return slot_tab, gate_tab


def fixed_hist(idx, n_buckets):
    """terrace/ta2a_fwd.py:318-321."""
    out = torch.zeros(n_buckets, dtype=torch.int64)
    return out if idx.numel() == 0 else out.scatter_add_(0, idx, torch.ones_like(idx))


def stable_argsort_small(key, n_buckets):
    """terrace/ta2a_fwd.py:338-345: composite float32 key bucket*n + position."""
    n = key.numel()
    if n_buckets * n >= (1 << 24):
        return torch.argsort(key, stable=True)
    return torch.argsort(torch.add(torch.arange(n, dtype=torch.float32), key.to(torch.float32), alpha=float(n)))


def k2_pack(x, expert_idx, gates, world, n_experts, rpn, groups_m):
    """terrace/ops/k2_ref.py:70-134 = plan + x[u_src] + the quota wire planes."""
    k = expert_idx.shape[1]
    slots = (n_experts // world) * rpn
    u_src, u_node, counts, inverse = plan(expert_idx, world, n_experts, rpn, groups_m)
    payload = x[u_src]
    mask, gate_rows = pack_quota_wire(expert_idx, gates, inverse, u_src.numel(), slots, k // groups_m)
    return payload, mask, gate_rows, u_src, counts, inverse


def k1_arrival(rx, rslot, rgate, quota, epr, rpn):
    """terrace/ops/__init__.py:287-299 (= terrace/ta2a_fwd.py:605-628 on the quota branch)."""
    flat = rslot.reshape(-1)
    owner = torch.div(flat, epr, rounding_mode="floor")
    ordo = stable_argsort_small(owner, rpn)
    r_idx = torch.div(ordo, quota, rounding_mode="floor")
    return rx[r_idx], rgate.reshape(-1)[ordo], r_idx, flat[ordo], fixed_hist(owner, rpn), ordo


def regroup(node_rx, my_slot, epr, capacity=None):
    """terrace/ta2a_fwd.py:641-646; with a capacity, this build's own rule (first `capacity` rows per expert)."""
    order = stable_argsort_small(my_slot, epr)
    counts = fixed_hist(my_slot, epr)
    if capacity is None:
        place = torch.empty_like(order)
        place[order] = torch.arange(order.numel())
        return node_rx[order], place, counts
    start = torch.cumsum(counts, 0) - counts
    rank = torch.empty_like(order)
    rank[order] = torch.arange(order.numel()) - start[my_slot[order]]
    kept = rank < capacity
    place = torch.where(kept, my_slot * capacity + rank, torch.full_like(rank, -1))
    padded = torch.zeros((epr * capacity, node_rx.shape[1]), dtype=node_rx.dtype)
    padded[place[kept]] = node_rx[kept]
    return padded, place, counts


def combine_two_level(ye, place, r_idx, gate_pairs, u_src, R, T):
    """terrace/ta2a_fwd.py:658-670: un-permute, gate-weighted index_add_ per send row, index_add per token.
    ``ye`` is in expert order ([places, H]), ``place`` names each arrival row's place there; a dropped row
    (place -1) contributes nothing."""
    ok = place >= 0
    ret = torch.zeros((place.numel(), ye.shape[1]), dtype=ye.dtype)
    ret[ok] = ye[place[ok]]
    red = torch.zeros((R, ye.shape[1]), dtype=ye.dtype)
    red.index_add_(0, r_idx, ret * gate_pairs.unsqueeze(1).to(ret.dtype))
    y = torch.zeros((T, ye.shape[1]), dtype=ye.dtype)
    return y.index_add(0, u_src, red)
