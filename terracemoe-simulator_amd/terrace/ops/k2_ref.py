"""terrace.ops.k2_ref: the name under which the reference keeps the executable specification of the send-side
chain (terrace/ops/k2_ref.py:70-134 there, a composition of torch operators).

This build has one implementation of that specification -- the kernels behind ``terrace.ops.k2_pack`` -- so
``k2_pack_ref`` resolves to them, with the reference function's own refusals in front: the same exception
classes for the same malformed calls, including the two it alone makes (more than 63 expert slots per node, and
an expert id outside ``[0, n_experts)`` on every call rather than on the guard's cadence).
"""
from __future__ import annotations

import torch

from .. import _hip
from . import TerraceK2PackFn, _check_k2, _require, k2_pack_raw


def k2_pack_ref(hidden: torch.Tensor, expert_idx: torch.Tensor, gates: torch.Tensor, world: int, n_experts: int,
                rpn: int, groups_m: int):
    """(payload [T*M, H], mask [T*M, q] int64 ascending slot ids, gate_rows [T*M, q], u_src [T*M] int64,
    node_counts [n_nodes] int64); ``payload`` and ``gate_rows`` carry gradients."""
    _require()
    _hip.need_device(hidden, expert_idx, gates)
    _check_k2(hidden, expert_idx, gates, world, n_experts, rpn, groups_m)
    slots = (n_experts // world) * rpn
    if slots > 63:
        raise ValueError(f"{slots} expert slots per node exceeds the chain bound")
    if torch.is_grad_enabled() and (hidden.requires_grad or gates.requires_grad):
        out = TerraceK2PackFn.apply(hidden, expert_idx, gates, world, n_experts, rpn, groups_m)
        return out
    out, ex = k2_pack_raw(hidden, expert_idx, gates, world, n_experts, rpn, groups_m, extras=True)
    if expert_idx.numel() and int(ex["status"][0]) & _hip.FAULT_ID_RANGE:
        raise ValueError("k2_pack_ref: expert id out of range")
    return out
