"""T-A2A dispatch plan on MI355X: the dedup'd, node-ordered send index.

Same interface as the reference module (terrace/ta2a.py there): ``plan_ta2a`` and
``dispatch_stats``, plus the ``_VERIFIED`` / ``_VERIFY_COUNT`` guard state tests may clear.
"""
from __future__ import annotations

import torch

from . import _hip
from . import ops as _ops

# (T, k, n_nodes, M) shapes whose fan-out / quota have been read back from the device, and
# per-shape call counters: the guard fires on the first call and on every 256th.
_VERIFIED: set = set()
_VERIFY_COUNT: dict = {}


def _raise_from_status(status: torch.Tensor, T: int, k: int, groups_m: int):
    """Reads the status words (one device->host sync) and raises what the reference's guard
    raises (terrace/ta2a.py:170-204 there)."""
    fault, occupied, off_quota, _ = status.tolist()
    n_rows = T * groups_m
    if fault & _hip.FAULT_ID_RANGE:
        raise ValueError("plan_ta2a: expert id out of range")
    if occupied != n_rows:
        raise ValueError(
            f"groups_m={groups_m} implies {n_rows} dispatch rows for T={T}, but the routing actually "
            f"produces {occupied} (fan-out {occupied / max(T, 1):.4f} != {groups_m}). Pass groups_m only "
            f"for routings with an exact fan-out; leave it None otherwise.")
    if off_quota:
        raise ValueError(
            f"groups_m={groups_m} requires every touched node to hold exactly k/M={k // groups_m} of a "
            f"token's experts, but {off_quota} (token, node) pairs violate the quota (e.g. a 3/1 split "
            f"with fan-out still == M). This routing is group-limited but not equal-quota; pass groups_m "
            f"only for equal-quota routings (t_route mode='full'/'quota_only'), leave it None otherwise.")


def _guard_due(key) -> bool:
    """Counts one call of shape ``key`` and says whether the guard reads the status words back on it."""
    cnt = _VERIFY_COUNT.get(key, 0)
    _VERIFY_COUNT[key] = cnt + 1
    return key not in _VERIFIED or cnt % 256 == 0


def _guard(status, T, k, n_nodes, groups_m):
    key = (T, k, n_nodes, groups_m)
    if _guard_due(key):
        _raise_from_status(status, T, k, groups_m)
        _VERIFIED.add(key)


def plan_ta2a(expert_idx: torch.Tensor, world: int, n_experts: int, rpn: int = 8,
              groups_m: int | None = None):
    """Build the dedup'd, node-ordered dispatch plan.  No collectives, no host sync except
    when the guard fires (first call per shape and every 256th).

    Returns
      u_src   [S] token index of each send row, S = T*groups_m
      u_node  [S] destination node of each row, ascending
      counts  [n_nodes] rows per destination node
      inverse [T*k] for each (token, expert) slot, the send row that carries it
    Rows are ordered (node ascending, token ascending).

    Without ``groups_m`` the fan-out is data dependent: S is read back from the device (one
    sync, as in the reference) and nothing is verified.  With it, S = T*groups_m is known up
    front and the equal-quota guard applies.
    """
    _hip.need_device(expert_idx)
    if expert_idx.dim() != 2:
        raise ValueError("plan_ta2a: expert_idx must be [T, k]")
    T, k = expert_idx.shape
    n_nodes = world // rpn
    if n_nodes * T >= (1 << 24):
        raise ValueError(
            f"plan_ta2a float32 key range exceeded: n_nodes*T = {n_nodes * T} >= 2^24; "
            f"shard tokens below {(1 << 24) // max(n_nodes, 1)} per rank or extend the "
            f"plan to int64 keys first")
    if world % rpn or n_experts % world:
        raise ValueError(f"plan_ta2a: world={world} rpn={rpn} n_experts={n_experts} not divisible")
    if groups_m is None:
        return _ops.plan_general(expert_idx.to(torch.int64), world, n_experts, rpn)
    if k % groups_m:
        raise ValueError(f"groups_m={groups_m} does not divide k={k}: the structured path's per-node quota "
                         f"k/M is not an integer. Leave groups_m None.")
    u_src, u_node, counts, inverse, _mask, status = _ops.plan_raw(
        expert_idx.to(torch.int64), world, n_experts, rpn, groups_m)
    _guard(status, T, k, n_nodes, groups_m)
    return u_src, u_node, counts, inverse


def dispatch_stats(expert_idx, world: int, n_experts: int, rpn: int = 8, groups_m: int | None = None):
    """Byte/message accounting for one dispatch, baseline vs T-A2A (terrace/ta2a.py:278-298)."""
    T, k = expert_idx.shape
    n_nodes = world // rpn
    _, _, counts, _ = plan_ta2a(expert_idx, world, n_experts, rpn, groups_m)
    rows_ta2a = int(counts.sum())
    return {"rows_baseline": T * k, "rows_ta2a": rows_ta2a, "dedup_x": (T * k) / max(rows_ta2a, 1),
            "msgs_baseline": world, "msgs_ta2a": n_nodes, "msg_growth_x": rpn}
