"""terrace.ops: loader switch and operator entry points of the MI355X kernel library.

Mirrors the reference plugin boundary (terrace/ops/__init__.py:53-179 there): the same
``TERRACE_CUSTOM_OPS`` / ``TERRACE_OPS_LIB`` environment switch read once and cached,
``status() / custom_ops_enabled() / reset()``, ``OpsState``, ``OpsLoadError``, and the
operators ``passthrough``, ``k1_arrival``, ``k1_arrival_segment`` plus ``k2_pack`` -- also
registered as ``torch.ops.terrace.{passthrough,k1_arrival,k2_pack}`` with the reference
schemas (terrace/ops/csrc/terrace_ops.cpp:230-232, terrace/ops/csrc/terrace_k2_pack.cpp:209-211).

One deliberate difference: this build contains no composed torch chain to fall back to, so
the library is the only implementation.  Switch values:

    unset, "1"       load the library; a failure is logged once as a WARNING and every
                     operator then raises OpsLoadError when called (never a silent fallback)
    "require" / "2"  a load failure raises RuntimeError from status()
    "0"              explicitly off: no load attempt, operators raise OpsLoadError
"""
from __future__ import annotations

import logging
import os
from dataclasses import dataclass

import torch

from .. import _hip

_LOG = logging.getLogger("terrace.ops")

_ENV_SWITCH = "TERRACE_CUSTOM_OPS"
_ENV_LIB = _hip.ENV_LIB
_REQUIRED_OPS = ("passthrough", "k1_arrival")


class OpsLoadError(RuntimeError):
    """The kernel library failed to load (.so not found / dlopen failed / symbol missing)."""


@dataclass(frozen=True)
class OpsState:
    requested: str        # "0" | "1" | "require" (normalised)
    loaded: bool
    lib: str | None
    reason: str           # "ok" when loaded


_STATE: OpsState | None = None


def _normalized_switch() -> str:
    raw = os.environ.get(_ENV_SWITCH, "1").strip()
    if raw in ("2", "require"):
        return "require"
    if raw == "0":
        return "0"
    return "1"


def _initialize() -> OpsState:
    switch = _normalized_switch()
    if switch == "0":
        return OpsState("0", False, None, f"{_ENV_SWITCH}=0 (explicitly off; no load attempted)")
    try:
        _hip.load()
        _register_torch_ops()
        _LOG.info("terrace kernel library loaded: %s", _hip.library_path())
        return OpsState(switch, True, _hip.library_path(), "ok")
    except _hip.LibraryError as e:
        if switch == "require":
            raise RuntimeError(f"{_ENV_SWITCH}={os.environ.get(_ENV_SWITCH)} requires the kernel library, "
                               f"but loading failed: {e}") from e
        _LOG.warning("terrace kernel library unavailable (%s) -- operators will raise when called", e)
        return OpsState(switch, False, None, str(e))


def status() -> OpsState:
    global _STATE
    if _STATE is None:
        _STATE = _initialize()
    return _STATE


def custom_ops_enabled() -> bool:
    return status().loaded


def reset() -> None:
    """Forget the cached verdict (test hook); the next status() re-reads the environment."""
    global _STATE
    _STATE = None
    _hip.unload_for_tests()


def _require():
    st = status()
    if not st.loaded:
        raise OpsLoadError(f"terrace kernel library not loaded: {st.reason}")


# --------------------------------------------------------------------------------------
# raw operators (forward only, no autograd)
# --------------------------------------------------------------------------------------

def _check_k1(rx, rslot, rgate, quota, epr, rpn, my_local):
    """Same refusals as the reference binding (terrace/ops/csrc/terrace_ops.cpp:123-144),
    minus its NPU-only limits (63 slots, 32-byte rows)."""
    if (rx is not None and rx.dim() != 2) or rslot.dim() != 2 or rgate.dim() != 2:
        raise RuntimeError("terrace::k1_arrival: rx/rslot/rgate must be 2-D")
    if rslot.dtype != torch.int64:
        raise RuntimeError("terrace::k1_arrival: rslot must be int64 (quota wire format)")
    if rx is not None and rgate.dtype != rx.dtype and rx.dtype != torch.uint8:
        raise RuntimeError("terrace::k1_arrival: rgate dtype must equal rx dtype (the gate plane is "
                           "allocated from the payload)")
    n_rows = rslot.shape[0] if rx is None else rx.shape[0]
    if not (rslot.shape[1] == quota and rgate.shape[1] == quota and rslot.shape[0] == n_rows
            and rgate.shape[0] == n_rows):
        raise RuntimeError(f"terrace::k1_arrival: geometry mismatch (rx "
                           f"{None if rx is None else tuple(rx.shape)}, rslot "
                           f"{tuple(rslot.shape)}, rgate {tuple(rgate.shape)}, quota {quota})")
    if not (quota > 0 and epr > 0 and rpn > 0 and 0 <= my_local < rpn):
        raise RuntimeError("terrace::k1_arrival: bad geometry scalars")
    if rgate.element_size() not in (2, 4):
        raise RuntimeError(f"terrace::k1_arrival: unsupported gate dtype {rgate.dtype}")


def k1_arrival_raw(rx, rslot, rgate, quota, epr, rpn, my_local=0, want_pair_pos=False, status_out=None,
                   workspace_out=None, tags=None, tags_out=None):
    """(send_buf, gate_pairs, r_idx, slot_idx, i_send[, pair_pos]) -- one library call.

    ``rx`` None: the index planes only (``send_buf`` is None); the workspace, which then holds what
    :func:`k1_arrival_move` needs, is appended to the list ``workspace_out``.  ``tags`` ([P] int64, one per pair):
    the same values in arrival order are appended to the list ``tags_out``."""
    _require()
    _hip.need_device(rx, rslot, rgate)
    _check_k1(rx, rslot, rgate, quota, epr, rpn, my_local)
    rslot, rgate = rslot.contiguous(), rgate.contiguous()
    dev = rslot.device
    R = rslot.shape[0]
    P = R * quota
    send_buf, row_bytes = None, 0
    if rx is not None:
        rx = _hip.as_rows(rx)
        row_bytes = _hip.row_arg(rx)
        send_buf = _hip.empty_rows(P, rx)
    gate_pairs = torch.empty((P,), dtype=rgate.dtype, device=dev)
    r_idx = torch.empty((P,), dtype=torch.int64, device=dev)
    slot_idx = torch.empty((P,), dtype=torch.int64, device=dev)
    i_send = torch.empty((rpn,), dtype=torch.int64, device=dev)
    pair_pos = torch.empty((P,), dtype=torch.int64, device=dev) if want_pair_pos else None
    carried = None
    if tags is not None:
        tags = _tag_plane(tags, P, dev)
        carried = torch.empty((P,), dtype=torch.int64, device=dev)
    st = status_out if status_out is not None else _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_k1_arrival_workspace", R, quota, rpn), dev)
    _hip.call("terrace_k1_arrival", _hip.ptr(rx), _hip.ptr(rslot), _hip.ptr(rgate), R, row_bytes,
              rgate.element_size(), quota, epr, rpn, my_local, _hip.ptr(send_buf), _hip.ptr(gate_pairs),
              _hip.ptr(r_idx), _hip.ptr(slot_idx), _hip.ptr(i_send), _hip.ptr(pair_pos), _hip.ptr(tags),
              _hip.ptr(carried), _hip.ptr(st), _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    if workspace_out is not None:
        workspace_out.append(ws)
    if tags_out is not None:
        tags_out.append(carried)
    out = (send_buf, gate_pairs, r_idx, slot_idx, i_send)
    return out + (pair_pos,) if want_pair_pos else out


def _tag_plane(tags, n, dev):
    tags = tags.contiguous().reshape(-1)
    if tags.dtype != torch.int64 or tags.numel() != n or tags.device != dev:
        raise RuntimeError(f"tags must be an int64 plane of {n} entries on {dev}")
    return tags


def _table_plane(table):
    if table.dtype != torch.int64 or not table.is_contiguous():
        raise RuntimeError("the table the tags index must be a contiguous int64 tensor")
    return table


def k1_arrival_static(rx, rslot, rgate, quota, epr, rpn, my_local, out):
    """The arrival chain through the entry point that allocates nothing: ``out`` is the tuple of caller-made
    tensors (send_buf, gate_pairs, r_idx, slot_idx, i_send, pair_pos, status) it fills, and the scratch the kernels
    need is a fixed array inside the library (so calls on one GPU must not overlap).  Inputs must already be
    contiguous; nothing here creates a tensor.  Raises RuntimeError when the input is larger than that array holds."""
    _require()
    send_buf, gate_pairs, r_idx, slot_idx, i_send, pair_pos, st = out
    _hip.need_device(rx, rslot, rgate, *out)
    _check_k1(rx, rslot, rgate, quota, epr, rpn, my_local)
    if not all(t.is_contiguous() for t in (rx, rslot, rgate) + tuple(out)):
        raise RuntimeError("k1_arrival_static: every tensor must be contiguous (the call makes no copies)")
    R, P = rslot.shape[0], rslot.shape[0] * quota
    if (tuple(send_buf.shape) != (P, rx.shape[1]) or send_buf.dtype != rx.dtype or gate_pairs.numel() != P
            or gate_pairs.dtype != rgate.dtype or i_send.numel() != rpn or st.numel() < _hip.STATUS_WORDS
            or st.dtype != torch.int32
            or any(t.numel() != P or t.dtype != torch.int64 for t in (r_idx, slot_idx, pair_pos))
            or i_send.dtype != torch.int64):
        raise RuntimeError("k1_arrival_static: an output tensor has the wrong shape or dtype")
    _hip.call("terrace_k1_arrival_static", _hip.ptr(rx), _hip.ptr(rslot), _hip.ptr(rgate), R,
              rx.shape[1] * rx.element_size(), rgate.element_size(), quota, epr, rpn, my_local, _hip.ptr(send_buf),
              _hip.ptr(gate_pairs), _hip.ptr(r_idx), _hip.ptr(slot_idx), _hip.ptr(i_send), _hip.ptr(pair_pos),
              _hip.ptr(st), _hip.stream(rx.device))
    return out


def _check_k2(hidden, expert_idx, gates, world, n_experts, rpn, groups_m):
    """Refusals of terrace/ops/k2_ref.py:87-108 (same exception classes), minus the id-range
    read-back (reported through the status words instead) and the 63-slot mask bound."""
    if expert_idx.dim() != 2 or (hidden is not None and hidden.dim() != 2) or gates.dim() != 2:
        raise ValueError("k2_pack: hidden/expert_idx/gates must be 2-D")
    T, k = expert_idx.shape
    if (hidden is not None and hidden.shape[0] != T) or gates.shape != expert_idx.shape:
        raise ValueError(f"k2_pack: geometry mismatch (hidden {None if hidden is None else tuple(hidden.shape)}, "
                         f"expert_idx {tuple(expert_idx.shape)}, gates {tuple(gates.shape)})")
    if hidden is not None and gates.dtype != hidden.dtype and hidden.dtype != torch.uint8:
        raise RuntimeError(f"k2_pack: gates dtype {gates.dtype} != hidden dtype {hidden.dtype} -- the gate "
                           f"plane derives from the payload; cast at the caller")
    if gates.element_size() not in (2, 4):
        raise RuntimeError(f"k2_pack: unsupported gate dtype {gates.dtype}")
    if expert_idx.dtype != torch.int64:
        raise RuntimeError("k2_pack: expert_idx must be int64")
    if world <= 0 or rpn <= 0 or groups_m <= 0 or n_experts <= 0:
        raise ValueError("k2_pack: bad geometry scalars")
    if world % rpn or n_experts % world or k % groups_m:
        raise ValueError(f"k2_pack: world={world} rpn={rpn} n_experts={n_experts} k={k} "
                         f"groups_m={groups_m} not divisible")


def _k2_extras(T, k, n_nodes, groups_m, gate_dtype, dev, combine_table=False):
    """The send side's optional planes: what plan_ta2a returns beside u_src, and the combine's per-token tables.
    With ``combine_table`` also ``pair_src`` (entry t*k+s behind each Hop-A pair) and ``where`` [T, k], the
    combine's place table, which the send side only pre-sets (-1) where a malformed routing leaves a rank without
    a pair: a later stage fills it through the pairs' tags."""
    i64 = dict(dtype=torch.int64, device=dev)
    ex = {"u_node": torch.empty((T * groups_m,), **i64), "inverse": torch.empty((T * k,), **i64),
          "node_offsets": torch.empty((n_nodes,), **i64), "pair_table": torch.empty((T, k), **i64),
          "sort_order": torch.empty((T, k), **i64), "token_rows": torch.empty((T, groups_m), **i64),
          "gate_sorted": torch.empty((T, k), dtype=gate_dtype, device=dev)}
    if combine_table:
        ex["pair_src"] = torch.empty((T * k,), **i64)
        ex["where"] = torch.empty((T, k), **i64)
    return ex


def k2_pack_raw(hidden, expert_idx, gates, world, n_experts, rpn, groups_m, extras=False, status_out=None,
                combine_table=False):
    """(payload, mask, gate_rows, u_src, node_counts) and, with ``extras``, a dict holding
    u_node, inverse, node_offsets, pair_table, sort_order, token_rows, gate_sorted and the
    status words (with ``combine_table`` also pair_src and the pre-set ``where`` table, see ``_k2_extras``).

    ``hidden`` None: the index planes only (``payload`` is None); ``extras["workspace"]`` then
    holds what :func:`k2_pack_move` needs."""
    _require()
    _hip.need_device(hidden, expert_idx, gates)
    _check_k2(hidden, expert_idx, gates, world, n_experts, rpn, groups_m)
    expert_idx, gates = expert_idx.contiguous(), gates.contiguous()
    dev = expert_idx.device
    T, k = expert_idx.shape
    S, q, n_nodes = T * groups_m, k // groups_m, world // rpn
    payload, row_bytes = None, 0
    if hidden is not None:
        hidden = _hip.as_rows(hidden)
        row_bytes = _hip.row_arg(hidden)
        payload = _hip.empty_rows(S, hidden)
    mask = torch.empty((S, q), dtype=torch.int64, device=dev)
    gate_rows = torch.empty((S, q), dtype=gates.dtype, device=dev)
    u_src = torch.empty((S,), dtype=torch.int64, device=dev)
    node_counts = torch.empty((n_nodes,), dtype=torch.int64, device=dev)
    ex = _k2_extras(T, k, n_nodes, groups_m, gates.dtype, dev, combine_table) if extras else {}
    st = status_out if status_out is not None else _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_k2_pack_workspace", T, k, n_nodes, groups_m), dev)
    _hip.call("terrace_k2_pack", _hip.ptr(hidden), _hip.ptr(expert_idx), _hip.ptr(gates), T,
              row_bytes, gates.element_size(), k, world, n_experts, rpn, groups_m,
              _hip.ptr(payload), _hip.ptr(mask), _hip.ptr(gate_rows), _hip.ptr(u_src), _hip.ptr(node_counts),
              _hip.ptr(ex.get("u_node")), _hip.ptr(ex.get("inverse")), _hip.ptr(ex.get("node_offsets")),
              _hip.ptr(ex.get("pair_table")), _hip.ptr(ex.get("sort_order")), _hip.ptr(ex.get("token_rows")),
              _hip.ptr(ex.get("gate_sorted")), _hip.ptr(ex.get("pair_src")), _hip.ptr(ex.get("where")), _hip.ptr(st),
              _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    out = (payload, mask, gate_rows, u_src, node_counts)
    if extras:
        ex["status"] = st
        if hidden is None:
            ex["workspace"] = ws
        return out, ex
    return out


def wire_words(quota: int, gate_bytes: int) -> int:
    """int64 words of one Hop-A small container row: ``quota`` slot ids, then ``quota`` gates padded to a word."""
    return quota + (quota * gate_bytes + 7) // 8


def k2_pack_wire(hidden, expert_idx, gates, world, n_experts, rpn, groups_m):
    """``k2_pack_raw(..., extras=True)`` with the slot-id and gate planes written by the kernel straight
    into the Hop-A small container: returns ((payload, mask, gate_rows, u_src, node_counts), extras) where
    ``extras["wire"]`` is the [T*M, W] int64 container and ``mask`` / ``gate_rows`` are views into it."""
    _require()
    _hip.need_device(hidden, expert_idx, gates)
    _check_k2(hidden, expert_idx, gates, world, n_experts, rpn, groups_m)
    hidden, expert_idx, gates = hidden.contiguous(), expert_idx.contiguous(), gates.contiguous()
    dev = expert_idx.device
    T, k = expert_idx.shape
    H = hidden.shape[1]
    S, q, n_nodes = T * groups_m, k // groups_m, world // rpn
    gb = gates.element_size()
    W = wire_words(q, gb)
    payload = torch.empty((S, H), dtype=hidden.dtype, device=dev)
    wire = torch.empty((S, W), dtype=torch.int64, device=dev)
    u_src = torch.empty((S,), dtype=torch.int64, device=dev)
    node_counts = torch.empty((n_nodes,), dtype=torch.int64, device=dev)
    ex = _k2_extras(T, k, n_nodes, groups_m, gates.dtype, dev)
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_k2_pack_workspace", T, k, n_nodes, groups_m), dev)
    _hip.call("terrace_k2_pack_wire", _hip.ptr(hidden), _hip.ptr(expert_idx), _hip.ptr(gates), T,
              H * hidden.element_size(), gb, k, world, n_experts, rpn, groups_m, _hip.ptr(payload), _hip.ptr(wire), W,
              _hip.ptr(u_src), _hip.ptr(node_counts), _hip.ptr(ex["u_node"]), _hip.ptr(ex["inverse"]),
              _hip.ptr(ex["node_offsets"]), _hip.ptr(ex["pair_table"]), _hip.ptr(ex["sort_order"]),
              _hip.ptr(ex["token_rows"]), _hip.ptr(ex["gate_sorted"]), _hip.ptr(st), _hip.ptr(ws), ws.numel(),
              _hip.stream(dev))
    per_word = 8 // gb
    mask = wire[:, :q]
    gate_rows = wire.view(gates.dtype)[:, q * per_word:q * per_word + q]
    ex["status"], ex["wire"] = st, wire
    return (payload, mask, gate_rows, u_src, node_counts), ex


def k1_arrival_wire(rx, rwire, gate_dtype, quota, epr, rpn, my_local=0, want_slot_idx=False):
    """The arrival chain reading an arrived Hop-A small container and writing the Hop-B container:
    (send_buf, meta [P,2] int64, r_idx, i_send, pair_pos); ``meta[:, 0]`` is slot_idx and the first
    element of word 1 (viewed in ``gate_dtype``) is gate_pairs.  ``want_slot_idx`` appends slot_idx as a dense [P]
    plane of its own (the same kernel writes it; a caller that needs it contiguous saves a strided copy)."""
    _require()
    _hip.need_device(rx, rwire)
    if rx.dim() != 2 or rwire.dim() != 2 or rwire.dtype != torch.int64 or rwire.shape[0] != rx.shape[0]:
        raise RuntimeError("terrace::k1_arrival: rx must be [R, H] and the container [R, W] int64")
    gb = torch.empty((), dtype=gate_dtype).element_size()
    if gb not in (2, 4) or rwire.shape[1] < wire_words(quota, gb):
        raise RuntimeError(f"terrace::k1_arrival: container rows of {rwire.shape[1]} words cannot hold quota {quota} "
                           f"ids and {gate_dtype} gates")
    if not (quota > 0 and epr > 0 and rpn > 0 and 0 <= my_local < rpn):
        raise RuntimeError("terrace::k1_arrival: bad geometry scalars")
    rx, rwire = rx.contiguous(), rwire.contiguous()
    dev = rx.device
    R, H = rx.shape
    P = R * quota
    send_buf = torch.empty((P, H), dtype=rx.dtype, device=dev)
    meta = torch.empty((P, 2), dtype=torch.int64, device=dev)
    r_idx = torch.empty((P,), dtype=torch.int64, device=dev)
    i_send = torch.empty((rpn,), dtype=torch.int64, device=dev)
    pair_pos = torch.empty((P,), dtype=torch.int64, device=dev)
    slot_idx = torch.empty((P,), dtype=torch.int64, device=dev) if want_slot_idx else None
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_k1_arrival_workspace", R, quota, rpn), dev)
    _hip.call("terrace_k1_arrival_wire", _hip.ptr(rx), _hip.ptr(rwire), rwire.shape[1], R, H * rx.element_size(), gb,
              quota, epr, rpn, my_local, _hip.ptr(send_buf), _hip.ptr(meta), _hip.ptr(r_idx),
              _hip.ptr(slot_idx) if want_slot_idx else None, None,
              _hip.ptr(i_send), _hip.ptr(pair_pos), _hip.ptr(st), _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    if want_slot_idx:
        return send_buf, meta, r_idx, i_send, pair_pos, slot_idx
    return send_buf, meta, r_idx, i_send, pair_pos


def regroup_wire(node_rx, my_meta, gate_dtype, epr, my_local=0):
    """Drop-less expert-order regroup reading slot ids and gates out of an arrived Hop-B container:
    (permuted, order, tokens_per_expert, place, permuted_gate)."""
    _require()
    _hip.need_device(node_rx, my_meta)
    if my_meta.dim() != 2 or my_meta.shape[1] != 2 or my_meta.dtype != torch.int64:
        raise RuntimeError("regroup: the Hop-B container must be [P, 2] int64")
    node_rx, my_meta = node_rx.contiguous(), my_meta.contiguous()
    dev = my_meta.device
    P = my_meta.shape[0]
    if node_rx.dim() != 2 or node_rx.shape[0] != P:
        raise RuntimeError(f"regroup: node_rx {tuple(node_rx.shape)} does not have one row per pair ({P})")
    gb = torch.empty((), dtype=gate_dtype).element_size()
    permuted = torch.empty_like(node_rx)
    pgate = torch.empty((P,), dtype=gate_dtype, device=dev)
    order = torch.empty((P,), dtype=torch.int64, device=dev)
    place = torch.empty((P,), dtype=torch.int64, device=dev)
    tpe = torch.empty((epr,), dtype=torch.int64, device=dev)
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_regroup_workspace", P, epr, -1), dev)
    _hip.call("terrace_regroup_wire", _hip.ptr(node_rx), _hip.ptr(my_meta), P, node_rx.shape[1] * node_rx.element_size(),
              gb, epr, my_local, -1, _hip.ptr(permuted), _hip.ptr(pgate), _hip.ptr(order), _hip.ptr(place), None,
              _hip.ptr(tpe), None, _hip.ptr(st), _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    return permuted, order, tpe, place, pgate


def plan_raw(expert_idx, world, n_experts, rpn, groups_m):
    """Index build only: (u_src, u_node, node_counts, inverse, extras incl. mask planes, status)."""
    _require()
    _hip.need_device(expert_idx)
    expert_idx = expert_idx.contiguous()
    dev = expert_idx.device
    T, k = expert_idx.shape
    S, q, n_nodes = T * groups_m, k // groups_m, world // rpn
    mask = torch.empty((S, q), dtype=torch.int64, device=dev)
    u_src = torch.empty((S,), dtype=torch.int64, device=dev)
    u_node = torch.empty((S,), dtype=torch.int64, device=dev)
    inverse = torch.empty((T * k,), dtype=torch.int64, device=dev)
    counts = torch.empty((n_nodes,), dtype=torch.int64, device=dev)
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_k2_pack_workspace", T, k, n_nodes, groups_m), dev)
    _hip.call("terrace_k2_pack", None, _hip.ptr(expert_idx), None, T, 0, 4, k, world, n_experts, rpn, groups_m,
              None, _hip.ptr(mask), None, _hip.ptr(u_src), _hip.ptr(counts), _hip.ptr(u_node),
              _hip.ptr(inverse), None, None, None, None, None, None, None, _hip.ptr(st), _hip.ptr(ws), ws.numel(),
              _hip.stream(dev))
    return u_src, u_node, counts, inverse, mask, st


def regroup(node_rx, my_slot, epr, my_local=0, capacity=None, my_gate=None, tags=None, table=None):
    """Expert-order regroup of the rows an expert card received.

    ``tags`` ([P] int64) with ``table`` (int64, any shape): ``table.view(-1)[tags[p]]`` is set to the place of
    row p (-1 when dropped), in place.

    Drop-less (``capacity=None``; terrace/ta2a_fwd.py:641-646 of the reference):
    returns ``(permuted, order, tokens_per_expert)`` (+ ``permuted_gate`` when ``my_gate``).
    With ``capacity`` (this build's own definition): expert x keeps its first ``capacity``
    rows in stable order; returns ``(padded [epr*capacity, H], dest [P], kept [P] bool,
    tokens_per_expert, kept_per_expert)`` (+ ``padded_gate``).
    """
    _require()
    _hip.need_device(node_rx, my_slot, my_gate)
    if my_slot.dtype != torch.int64:
        raise RuntimeError("regroup: my_slot must be int64")
    my_slot = my_slot.contiguous().reshape(-1)
    dev = my_slot.device
    P = my_slot.numel()
    if node_rx.dim() != 2 or node_rx.shape[0] != P:
        raise RuntimeError(f"regroup: node_rx {tuple(node_rx.shape)} does not have one row per slot id ({P})")
    node_rx = _hip.as_rows(node_rx)
    cap = -1 if capacity is None else int(capacity)
    places = P if capacity is None else epr * cap
    permuted = _hip.empty_rows(places, node_rx)
    tpe = torch.empty((epr,), dtype=torch.int64, device=dev)
    kpe = torch.empty((epr,), dtype=torch.int64, device=dev)
    order = torch.empty((P,), dtype=torch.int64, device=dev) if capacity is None else None
    dest = torch.empty((P,), dtype=torch.int64, device=dev) if capacity is not None else None
    kept = torch.empty((P,), dtype=torch.uint8, device=dev) if capacity is not None else None
    pgate = None
    gate_bytes = 4
    if my_gate is not None:
        my_gate = my_gate.contiguous().reshape(-1)
        gate_bytes = my_gate.element_size()
        pgate = torch.empty((places,), dtype=my_gate.dtype, device=dev)
    n_tags = 0
    if tags is not None:
        tags, table = _tag_plane(tags, P, dev), _table_plane(table)
        n_tags = table.numel()
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_regroup_workspace", P, epr, cap), dev)
    _hip.call("terrace_regroup", _hip.ptr(node_rx), _hip.ptr(my_slot), _hip.ptr(my_gate), P,
              _hip.row_arg(node_rx), gate_bytes, epr, my_local, cap, _hip.ptr(permuted), _hip.ptr(pgate),
              _hip.ptr(order), _hip.ptr(dest), _hip.ptr(kept), _hip.ptr(tpe), _hip.ptr(kpe), _hip.ptr(tags),
              _hip.ptr(table), n_tags, _hip.ptr(st), _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    if capacity is None:
        out = (permuted, order, tpe)
    else:
        out = (permuted, dest, kept.view(torch.bool), tpe, kpe)
    return out + (pgate,) if my_gate is not None else out


def hopb_scatter(rx, rslot, rgate, quota, n_local, first_slot=0, capacity=None, want_pairs=False,
                 workspace_out=None, tags=None, table=None):
    """Hop-B local scatter in one pass: what ``k1_arrival`` followed by ``regroup(epr=n_local)`` produce when
    every slot the arrived rows name is local to this GPU, without the send buffer between them.

    Returns a dict: ``permuted`` ([P, H], or [n_local*capacity, H] with zero padding rows), ``place`` [P]
    (where pair ``p = r*quota + i`` sits in ``permuted``; -1 = dropped), ``kept`` [P] bool (None drop-less),
    ``tokens_per_expert`` / ``kept_per_expert`` [n_local], ``permuted_gate`` (the gate of each place, when
    ``rgate`` is given) and, with ``want_pairs``, ``pair_of_place`` (-1 on padding).

    ``rx`` None: the index planes only; the workspace :func:`hopb_scatter_move` needs is appended to
    ``workspace_out``.  ``tags`` ([P] int64) with ``table`` (int64): ``table.view(-1)[tags[p]] = place[p]``, in place."""
    _require()
    _hip.need_device(rx, rslot, rgate)
    if rslot.dim() != 2 or rslot.dtype != torch.int64 or rslot.shape[1] != quota:
        raise RuntimeError("hopb_scatter: rslot must be an int64 [R, quota] table")
    if rx is not None and (rx.dim() != 2 or rx.shape[0] != rslot.shape[0]):
        raise RuntimeError(f"hopb_scatter: rx {tuple(rx.shape)} does not have one row per row of rslot")
    if rgate is not None and (tuple(rgate.shape) != tuple(rslot.shape) or rgate.element_size() not in (2, 4)):
        raise RuntimeError("hopb_scatter: rgate must match rslot and hold 2- or 4-byte elements")
    if not (quota > 0 and n_local > 0 and first_slot >= 0):
        raise RuntimeError("hopb_scatter: bad geometry scalars")
    rslot = rslot.contiguous()
    dev = rslot.device
    R = rslot.shape[0]
    P = R * quota
    cap = -1 if capacity is None else int(capacity)
    places = P if capacity is None else n_local * cap
    i64 = dict(dtype=torch.int64, device=dev)
    permuted, row_bytes = None, 0
    if rx is not None:
        rx = _hip.as_rows(rx)
        row_bytes = _hip.row_arg(rx)
        permuted = _hip.empty_rows(places, rx)
    pgate, gate_bytes = None, 4
    if rgate is not None:
        rgate = rgate.contiguous()
        gate_bytes = rgate.element_size()
        pgate = torch.empty((places,), dtype=rgate.dtype, device=dev)
    place = torch.empty((P,), **i64)
    kept = torch.empty((P,), dtype=torch.uint8, device=dev) if capacity is not None else None
    pairs = torch.empty((places,), **i64) if want_pairs else None
    tpe, kpe = torch.empty((n_local,), **i64), torch.empty((n_local,), **i64)
    n_tags = 0
    if tags is not None:
        tags, table = _tag_plane(tags, P, dev), _table_plane(table)
        n_tags = table.numel()
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_hopb_scatter_workspace", R, quota, n_local), dev)
    _hip.call("terrace_hopb_scatter", _hip.ptr(rx), _hip.ptr(rslot), _hip.ptr(rgate), R, row_bytes, gate_bytes, quota,
              first_slot, n_local, cap, _hip.ptr(permuted), _hip.ptr(pgate), _hip.ptr(place), _hip.ptr(kept),
              _hip.ptr(pairs), _hip.ptr(tpe), _hip.ptr(kpe), _hip.ptr(tags), _hip.ptr(table), n_tags, _hip.ptr(st),
              _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    if workspace_out is not None:
        workspace_out.append(ws)
    return {"permuted": permuted, "place": place, "kept": None if kept is None else kept.view(torch.bool),
            "tokens_per_expert": tpe, "kept_per_expert": kpe, "permuted_gate": pgate, "pair_of_place": pairs,
            "status": st}


def hopb_scatter_move(rx, workspace, quota, n_local, capacity=None):
    """Second phase of :func:`hopb_scatter` called with ``rx=None``: the expert-order buffer."""
    _require()
    _hip.need_device(rx, workspace)
    if rx.dim() != 2:
        raise RuntimeError("hopb_scatter: rx must be 2-D")
    rx = rx.contiguous()
    R, H = rx.shape
    cap = -1 if capacity is None else int(capacity)
    places = R * quota if capacity is None else n_local * cap
    permuted = torch.empty((places, H), dtype=rx.dtype, device=rx.device)
    _hip.call("terrace_hopb_scatter_move", _hip.ptr(rx), R, H * rx.element_size(), quota, n_local, cap,
              _hip.ptr(permuted), _hip.ptr(workspace), workspace.numel(), _hip.stream(rx.device))
    return permuted


# ---- the stage operators in two phases (index planes first, rows later) -----------------------------
def k2_pack_index(expert_idx, gates, world, n_experts, rpn, groups_m):
    """First phase of :func:`k2_pack_raw`: every index plane, no rows.  Returns
    ((mask, gate_rows, u_src, node_counts), extras) with ``extras["workspace"]`` holding what
    :func:`k2_pack_move` needs to move the rows later."""
    out, ex = k2_pack_raw(None, expert_idx, gates, world, n_experts, rpn, groups_m, extras=True)
    return out[1:], ex


def k2_pack_move(hidden, workspace, k, world, rpn, groups_m):
    """Second phase: the Hop-A payload [T*groups_m, H] of ``hidden`` from the first phase's workspace."""
    _require()
    _hip.need_device(hidden, workspace)
    if hidden.dim() != 2:
        raise ValueError("k2_pack: hidden must be 2-D")
    hidden = hidden.contiguous()
    T, H = hidden.shape
    payload = torch.empty((T * groups_m, H), dtype=hidden.dtype, device=hidden.device)
    _hip.call("terrace_k2_pack_move", _hip.ptr(hidden), T, H * hidden.element_size(), k, world // rpn, groups_m,
              _hip.ptr(payload), _hip.ptr(workspace), workspace.numel(), _hip.stream(hidden.device))
    return payload


def k1_arrival_index(rslot, rgate, quota, epr, rpn, my_local=0):
    """First phase of :func:`k1_arrival_raw`: (gate_pairs, r_idx, slot_idx, i_send, pair_pos, workspace)."""
    ws = []
    out = k1_arrival_raw(None, rslot, rgate, quota, epr, rpn, my_local, want_pair_pos=True, workspace_out=ws)
    return out[1:] + (ws[0],)


def k1_arrival_move(rx, workspace, quota, rpn):
    """Second phase: ``send_buf`` [R*quota, H] of the arrived rows ``rx`` from the first phase's workspace."""
    _require()
    _hip.need_device(rx, workspace)
    if rx.dim() != 2:
        raise RuntimeError("k1_arrival: rx must be 2-D")
    rx = rx.contiguous()
    R, H = rx.shape
    send_buf = torch.empty((R * quota, H), dtype=rx.dtype, device=rx.device)
    _hip.call("terrace_k1_arrival_move", _hip.ptr(rx), R, H * rx.element_size(), quota, rpn, _hip.ptr(send_buf),
              _hip.ptr(workspace), workspace.numel(), _hip.stream(rx.device))
    return send_buf


def regroup_index(my_slot, epr, my_local=0, capacity=None):
    """First phase of :func:`regroup`: a dict with tokens_per_expert, kept_per_expert, the row -> place plane
    ``dest`` (-1 = dropped), ``order`` (drop-less) or ``kept`` (capacity), and the workspace."""
    _require()
    _hip.need_device(my_slot)
    if my_slot.dtype != torch.int64:
        raise RuntimeError("regroup: my_slot must be int64")
    my_slot = my_slot.contiguous().reshape(-1)
    dev = my_slot.device
    P = my_slot.numel()
    cap = -1 if capacity is None else int(capacity)
    i64 = dict(dtype=torch.int64, device=dev)
    tpe, kpe, dest = torch.empty((epr,), **i64), torch.empty((epr,), **i64), torch.empty((P,), **i64)
    order = torch.empty((P,), **i64) if capacity is None else None
    kept = torch.empty((P,), dtype=torch.uint8, device=dev) if capacity is not None else None
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_regroup_workspace", P, epr, cap), dev)
    _hip.call("terrace_regroup", None, _hip.ptr(my_slot), None, P, 0, 4, epr, my_local, cap, None, None,
              _hip.ptr(order), _hip.ptr(dest), _hip.ptr(kept), _hip.ptr(tpe), _hip.ptr(kpe), None, None, 0,
              _hip.ptr(st), _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    return {"tokens_per_expert": tpe, "kept_per_expert": kpe, "dest": dest, "order": order,
            "kept": None if kept is None else kept.view(torch.bool), "workspace": ws}


def regroup_move(node_rx, workspace, epr, capacity=None):
    """Second phase: the expert-order buffer ([P, H], or [epr*capacity, H] with zero padding rows)."""
    _require()
    _hip.need_device(node_rx, workspace)
    if node_rx.dim() != 2:
        raise RuntimeError("regroup: node_rx must be 2-D")
    node_rx = node_rx.contiguous()
    P, H = node_rx.shape
    cap = -1 if capacity is None else int(capacity)
    places = P if capacity is None else epr * cap
    permuted = torch.empty((places, H), dtype=node_rx.dtype, device=node_rx.device)
    _hip.call("terrace_regroup_move", _hip.ptr(node_rx), P, H * node_rx.element_size(), epr, cap,
              _hip.ptr(permuted), _hip.ptr(workspace), workspace.numel(), _hip.stream(node_rx.device))
    return permuted


def gather_rows(src, idx):
    """``src[idx]`` for a 2-D ``src``; indices outside ``[0, len(src))`` (negative ones included) give
    zero rows -- the kernel never forms an address from them."""
    _require()
    _hip.need_device(src, idx)
    src, idx = (_hip.as_rows(src) if src.dim() == 2 else src.contiguous()), idx.contiguous().reshape(-1)
    if idx.dtype != torch.int64:
        raise RuntimeError("gather_rows: idx must be int64")
    if src.dim() == 2 and not src.is_contiguous():          # rows on a pitch: the output takes the same pitch
        out = _hip.empty_rows(idx.numel(), src)
        row_bytes = _hip.row_arg(src)
    else:
        out = torch.empty((idx.numel(),) + tuple(src.shape[1:]), dtype=src.dtype, device=src.device)
        row_bytes = src.element_size()
        for d in src.shape[1:]:
            row_bytes *= int(d)
    _hip.call("terrace_gather_rows", _hip.ptr(src), src.shape[0], _hip.ptr(idx), idx.numel(), row_bytes,
              _hip.ptr(out), _hip.stream(src.device))
    return out


def scatter_rows(src, pos, n_dst):
    """``dst[pos[r, f]] = src[r]``: each source row is read once and written ``pos.shape[1]``
    times (places outside ``[0, n_dst)`` are skipped).  ``dst`` has ``n_dst`` rows; rows no place
    names are left uninitialised."""
    _require()
    _hip.need_device(src, pos)
    src, pos = (_hip.as_rows(src) if src.dim() == 2 else src.contiguous()), pos.contiguous()
    if pos.dtype != torch.int64 or pos.dim() != 2 or pos.shape[0] != src.shape[0]:
        raise RuntimeError("scatter_rows: pos must be int64 [n_src, fan]")
    if src.dim() == 2 and not src.is_contiguous():          # rows on a pitch: the output takes the same pitch
        dst = _hip.empty_rows(int(n_dst), src)
        row_bytes = _hip.row_arg(src)
    else:
        dst = torch.empty((n_dst,) + tuple(src.shape[1:]), dtype=src.dtype, device=src.device)
        row_bytes = src.element_size()
        for d in src.shape[1:]:
            row_bytes *= int(d)
    _hip.call("terrace_scatter_rows", _hip.ptr(src), _hip.ptr(pos), src.shape[0], pos.shape[1], row_bytes,
              _hip.ptr(dst), int(n_dst), _hip.stream(src.device))
    return dst


def index_chain(table, idx):
    """``table[idx]`` over int64 planes (entries outside the table, negative ones included, give -1)."""
    _require()
    _hip.need_device(table, idx)
    table, idx = table.contiguous(), idx.contiguous()
    out = torch.empty_like(idx)
    _hip.call("terrace_index_chain", _hip.ptr(table), table.numel(), _hip.ptr(idx), idx.numel(), _hip.ptr(out),
              _hip.stream(idx.device))
    return out


def index_chain2(outer, inner, idx):
    """``outer[inner[idx]]`` over int64 planes in one launch (an entry outside its table at either
    level, negative ones included, gives -1)."""
    _require()
    _hip.need_device(outer, inner, idx)
    outer, inner, idx = outer.contiguous(), inner.contiguous(), idx.contiguous()
    out = torch.empty_like(idx)
    _hip.call("terrace_index_chain2", _hip.ptr(outer), outer.numel(), _hip.ptr(inner), inner.numel(),
              _hip.ptr(idx), idx.numel(), _hip.ptr(out), _hip.stream(idx.device))
    return out


def combine(src, idx, weights=None, out_dtype=None, fp8_hidden=None):
    """``out[i] = sum_j weights[i,j] * src[idx[i,j]]`` accumulated in fp32 in the order ``idx``
    lists the rows, rounded once to ``out_dtype`` (default: ``src.dtype``, or bf16 for fp8 rows).

    ``src`` is [n, H] float32 / bfloat16 / float16, or with ``fp8_hidden=H`` a uint8
    [n, H + H/32] plane of e4m3 rows followed by their per-128 fp32 scales.
    """
    _require()
    _hip.need_device(src, idx, weights)
    src, idx = _hip.as_rows(src), idx.contiguous()
    if idx.dim() != 2 or idx.dtype != torch.int64:
        raise RuntimeError("combine: idx must be a 2-D int64 table")
    n_out, fan = idx.shape
    if fp8_hidden is not None:
        hidden = int(fp8_hidden)
        if src.dtype != torch.uint8 or src.shape[1] != hidden + hidden // 32 or hidden % 128:
            raise RuntimeError("combine: fp8 rows must be uint8 [n, H + H/32] with H a multiple of 128")
        src_code = _hip.FP8_B128
        out_dtype = out_dtype or torch.bfloat16
    else:
        hidden = src.shape[1]
        src_code = _hip.float_code(src.dtype)
        out_dtype = out_dtype or src.dtype
    w_code = 0
    if weights is not None:
        weights = weights.contiguous()
        if tuple(weights.shape) != (n_out, fan):
            raise RuntimeError("combine: weights must match idx")
        w_code = _hip.float_code(weights.dtype)
    out = torch.empty((n_out, hidden), dtype=out_dtype, device=src.device)
    pitch = 0 if src.is_contiguous() else src.stride(0) * src.element_size()
    _hip.call("terrace_combine_pitched", _hip.ptr(src), src.shape[0], src_code, pitch, _hip.ptr(idx), _hip.ptr(weights),
              w_code, n_out, fan, hidden, _hip.ptr(out), _hip.float_code(out_dtype), _hip.stream(src.device))
    return out


def combine_two_level(src, inner, outer, out_dtype=None):
    """``combine(combine(src, inner, out_dtype=src.dtype), outer, out_dtype=out_dtype)`` -- the reference's two
    ``index_add`` levels, each an fp32 sum rounded once -- bit for bit, in one pass when the shape allows it (the
    ``[len(inner), H]`` plane between the levels is then never written): float rows that are 16-byte multiples and an
    inner table 1, 2, 4 or 8 ids wide; any other shape runs the two levels one after the other."""
    _require()
    _hip.need_device(src, inner, outer)
    if inner.dim() != 2 or outer.dim() != 2 or inner.dtype != torch.int64 or outer.dtype != torch.int64:
        raise RuntimeError("combine_two_level: inner and outer must be 2-D int64 tables")
    out_dtype = out_dtype or src.dtype
    fused = (src.dim() == 2 and src.is_contiguous() and src.dtype in (torch.float32, torch.bfloat16, torch.float16)
             and out_dtype in (torch.float32, torch.bfloat16, torch.float16)
             and inner.shape[1] in (1, 2, 4, 8) and outer.shape[1] >= 1
             and (src.shape[1] * src.element_size()) % 16 == 0
             and (src.shape[1] * torch.empty((), dtype=out_dtype).element_size()) % 16 == 0
             and src.data_ptr() % 16 == 0)
    if not fused:
        return combine(combine(src, inner, None, out_dtype=src.dtype), outer, None, out_dtype=out_dtype)
    inner, outer = inner.contiguous(), outer.contiguous()
    out = torch.empty((outer.shape[0], src.shape[1]), dtype=out_dtype, device=src.device)
    _hip.call("terrace_combine_two_level", _hip.ptr(src), src.shape[0], _hip.float_code(src.dtype), _hip.ptr(inner),
              inner.shape[0], inner.shape[1], _hip.ptr(outer), outer.shape[0], outer.shape[1], src.shape[1],
              _hip.ptr(out), _hip.float_code(out_dtype), _hip.stream(src.device))
    return out


def hist(idx, n_buckets, as_float=False):
    _require()
    _hip.need_device(idx)
    idx = idx.contiguous().reshape(-1)
    if idx.dtype != torch.int64:
        raise RuntimeError("hist: idx must be int64")
    dev = idx.device
    out = torch.empty((n_buckets,), dtype=torch.float32 if as_float else torch.int64, device=dev)
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_hist_workspace", idx.numel(), n_buckets), dev)
    _hip.call("terrace_hist", _hip.ptr(idx), idx.numel(), n_buckets, _hip.ptr(out), int(as_float), _hip.ptr(st),
              _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    return out, st


def argsort_small(key, n_buckets):
    _require()
    _hip.need_device(key)
    key = key.contiguous().reshape(-1)
    if key.dtype != torch.int64:
        raise RuntimeError("argsort_small: key must be int64")
    dev = key.device
    order = torch.empty_like(key)
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_argsort_small_workspace", key.numel(), n_buckets), dev)
    _hip.call("terrace_argsort_small", _hip.ptr(key), key.numel(), n_buckets, _hip.ptr(order), None, _hip.ptr(st),
              _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    return order, st


def plan_general(expert_idx, world, n_experts, rpn):
    """plan_ta2a with a data-dependent fan-out: (u_src [S], u_node [S], counts, inverse [T*k]);
    S = counts.sum() is read back (the one synchronisation the reference pays too)."""
    _require()
    _hip.need_device(expert_idx)
    expert_idx = expert_idx.contiguous()
    dev = expert_idx.device
    T, k = expert_idx.shape
    n_nodes = world // rpn
    cap = T * min(k, n_nodes)
    u_src = torch.empty((cap,), dtype=torch.int64, device=dev)
    u_node = torch.empty((cap,), dtype=torch.int64, device=dev)
    inverse = torch.empty((T * k,), dtype=torch.int64, device=dev)
    # the counts and the status block share one allocation, so that one copy to the host brings both
    words = _hip.STATUS_WORDS // 2
    both = torch.empty((n_nodes + words,), dtype=torch.int64, device=dev)
    counts, st = both[:n_nodes], both[n_nodes:].view(torch.int32)
    ws = _hip.workspace(_hip.query("terrace_plan_general_workspace", T, k, n_nodes), dev)
    _hip.call("terrace_plan_general", _hip.ptr(expert_idx), T, k, world, n_experts, rpn, _hip.ptr(u_src),
              _hip.ptr(u_node), _hip.ptr(counts), _hip.ptr(inverse), _hip.ptr(st), _hip.ptr(ws), ws.numel(),
              _hip.stream(dev))
    host = both.tolist()
    if (host[n_nodes] & 0xFFFFFFFF) & _hip.FAULT_ID_RANGE:           # status word 0: the low half of the first word
        raise ValueError("plan_ta2a: expert id out of range")
    n_rows = sum(host[:n_nodes])
    return u_src[:n_rows], u_node[:n_rows], counts, inverse


def build_mask(expert_idx, inverse, n_rows, slots):
    """Per-send-row int64 bitmask: bit j of row r set iff node-local slot j wants the row."""
    _require()
    _hip.need_device(expert_idx, inverse)
    e, inv = expert_idx.contiguous().reshape(-1), inverse.contiguous().reshape(-1)
    if e.dtype != torch.int64 or inv.dtype != torch.int64 or e.numel() != inv.numel():
        raise RuntimeError("build_mask: expert_idx and inverse must be int64 planes of equal size")
    dev = e.device
    mask = torch.zeros((n_rows,), dtype=torch.int64, device=dev)
    st = torch.zeros(_hip.STATUS_WORDS, dtype=torch.int32, device=dev)
    _hip.call("terrace_build_mask", _hip.ptr(e), _hip.ptr(inv), e.numel(), slots, n_rows, _hip.ptr(mask),
              _hip.ptr(st), _hip.stream(dev))
    return mask, st


def scatter_elems(vals, rows, cols, out, col_mod=0):
    """``out[rows[i], c] = vals[i]`` in place on a dense 2-D ``out`` with ``c = cols[i]``, or
    ``cols[i] % col_mod`` when ``col_mod > 0``; returns ``out``."""
    _require()
    _hip.need_device(vals, rows, cols, out)
    vals, rows, cols = vals.contiguous().reshape(-1), rows.contiguous().reshape(-1), cols.contiguous().reshape(-1)
    if vals.dtype != out.dtype or not out.is_contiguous() or out.dim() != 2:
        raise RuntimeError("scatter_elems: out must be a dense 2-D plane of the values' dtype")
    if rows.dtype != torch.int64 or cols.dtype != torch.int64 or not (vals.numel() == rows.numel() == cols.numel()):
        raise RuntimeError("scatter_elems: rows/cols must be int64 planes as long as vals")
    _hip.call("terrace_scatter_elems", _hip.ptr(vals), vals.element_size(), _hip.ptr(rows), _hip.ptr(cols),
              int(col_mod), vals.numel(), out.shape[0], out.shape[1], _hip.ptr(out), _hip.stream(out.device))
    return out


def expand_mask(rmask, slots, quota=None):
    """(r_idx, slot_idx) demand pairs of arrived bitmasks; without a quota the pair count is
    read back from the device (the data-dependent shape ``nonzero`` has in the reference)."""
    _require()
    _hip.need_device(rmask)
    rmask = rmask.contiguous().reshape(-1)
    if rmask.dtype != torch.int64:
        raise RuntimeError("expand_mask: rmask must be int64")
    dev = rmask.device
    R = rmask.numel()
    if quota is not None:
        r_idx = torch.empty((R * quota,), dtype=torch.int64, device=dev)
        slot_idx = torch.empty((R * quota,), dtype=torch.int64, device=dev)
        _hip.call("terrace_expand_mask_quota", _hip.ptr(rmask), R, slots, quota, _hip.ptr(r_idx), _hip.ptr(slot_idx),
                  _hip.stream(dev))
        return r_idx, slot_idx
    n_pairs = torch.empty((1,), dtype=torch.int64, device=dev)
    ws = _hip.workspace(_hip.query("terrace_expand_mask_workspace", R), dev)
    _hip.call("terrace_expand_mask_count", _hip.ptr(rmask), R, slots, _hip.ptr(n_pairs), _hip.ptr(ws), ws.numel(),
              _hip.stream(dev))
    P = int(n_pairs.item())
    r_idx = torch.empty((P,), dtype=torch.int64, device=dev)
    slot_idx = torch.empty((P,), dtype=torch.int64, device=dev)
    if P == 0:
        return r_idx, slot_idx
    _hip.call("terrace_expand_mask_fill", _hip.ptr(rmask), R, slots, _hip.ptr(r_idx), _hip.ptr(slot_idx),
              _hip.ptr(ws), _hip.stream(dev))
    return r_idx, slot_idx


def arrival_pairs(rx, r_in, slot_in, rgate, epr, rpn, move=True):
    """Arrival chain over an explicit pair list (the general branch):
    (send_buf, gate_pairs, r_idx, slot_idx, i_send, ordo) with pairs in stable owner-card order
    and ``gate_pairs = rgate[r_idx, slot_idx]`` looked up in the sparse [R, width] plane.

    ``move=False``: the index planes only (``send_buf`` is None), for a caller that moves the rows itself -- a scatter
    over the per-row table of ``r_idx`` reads each arrived row once, where this call's gather reads it once per pair."""
    _require()
    _hip.need_device(rx, r_in, slot_in, rgate)
    rx, r_in, slot_in = rx.contiguous(), r_in.contiguous().reshape(-1), slot_in.contiguous().reshape(-1)
    if r_in.dtype != torch.int64 or slot_in.dtype != torch.int64 or r_in.numel() != slot_in.numel():
        raise RuntimeError("arrival_pairs: r_idx/slot_idx must be int64 planes of equal length")
    if rx.dim() != 2:
        raise RuntimeError("arrival_pairs: rx must be 2-D")
    dev = rx.device
    R, H = rx.shape
    P = r_in.numel()
    gate_bytes, width, gate_pairs = 4, 0, None
    if rgate is not None:
        rgate = rgate.contiguous()
        if rgate.dim() != 2 or rgate.shape[0] != R or rgate.element_size() not in (2, 4):
            raise RuntimeError("arrival_pairs: rgate must be a [R, width] plane of 2- or 4-byte elements")
        gate_bytes, width = rgate.element_size(), rgate.shape[1]
        gate_pairs = torch.empty((P,), dtype=rgate.dtype, device=dev)
    send_buf = torch.empty((P, H), dtype=rx.dtype, device=dev) if move else None
    r_idx = torch.empty((P,), dtype=torch.int64, device=dev)
    slot_idx = torch.empty((P,), dtype=torch.int64, device=dev)
    ordo = torch.empty((P,), dtype=torch.int64, device=dev)
    i_send = torch.empty((rpn,), dtype=torch.int64, device=dev)
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_arrival_pairs_workspace", P, rpn), dev)
    _hip.call("terrace_arrival_pairs", _hip.ptr(rx) if move else None, _hip.ptr(r_in), _hip.ptr(slot_in), _hip.ptr(rgate), R, P,
              H * rx.element_size(), gate_bytes, width, epr, rpn, _hip.ptr(send_buf), _hip.ptr(gate_pairs),
              _hip.ptr(r_idx), _hip.ptr(slot_idx), _hip.ptr(i_send), _hip.ptr(ordo), _hip.ptr(st), _hip.ptr(ws),
              ws.numel(), _hip.stream(dev))
    return send_buf, gate_pairs, r_idx, slot_idx, i_send, ordo


def segment_table(seg, n_seg, width):
    """[n_seg, width] int64 table listing, per target s, the positions i with ``seg[i] == s`` in
    ascending order, padded with -1: ``combine(src, table)`` is then ``index_add`` by ``seg``."""
    _require()
    _hip.need_device(seg)
    seg = seg.contiguous().reshape(-1)
    if seg.dtype != torch.int64:
        raise RuntimeError("segment_table: seg must be int64")
    dev = seg.device
    table = torch.empty((n_seg, width), dtype=torch.int64, device=dev)
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_segment_table_workspace", n_seg), dev)
    _hip.call("terrace_segment_table", _hip.ptr(seg), seg.numel(), n_seg, width, _hip.ptr(table), _hip.ptr(st),
              _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    return table, st


def pair_places(order, r_idx, slot_idx, u_src, u_node, expert_idx, slots):
    """(where [T,k], token_of_place [P]): the place of every (token, expert) pair in the expert-order
    buffer and the token behind every place."""
    _require()
    _hip.need_device(order, r_idx, slot_idx, u_src, u_node, expert_idx)
    planes = [t.contiguous().reshape(-1) for t in (order, r_idx, slot_idx, u_src, u_node)]
    expert_idx = expert_idx.contiguous()
    if any(t.dtype != torch.int64 for t in planes) or expert_idx.dtype != torch.int64:
        raise RuntimeError("pair_places: every plane must be int64")
    order, r_idx, slot_idx, u_src, u_node = planes
    dev = expert_idx.device
    T, k = expert_idx.shape
    P = order.numel()
    where = torch.empty((T, k), dtype=torch.int64, device=dev)
    tok = torch.empty((P,), dtype=torch.int64, device=dev)
    st = _hip.new_status(dev)
    _hip.call("terrace_pair_places", _hip.ptr(order), _hip.ptr(r_idx), _hip.ptr(slot_idx), _hip.ptr(u_src),
              _hip.ptr(u_node), _hip.ptr(expert_idx), P, T, k, slots, u_src.numel(), _hip.ptr(where), _hip.ptr(tok),
              _hip.ptr(st), _hip.stream(dev))
    return where, tok


def routing_map_topk(routing_map, probs):
    """Dense [T,E] routing map -> ([T,k] ascending expert ids, [T,k] their probs).  One
    synchronisation (the per-row count's min and max), as in the reference; raises
    RuntimeError when rows do not all hold the same non-zero count."""
    _require()
    _hip.need_device(routing_map, probs)
    if routing_map.dim() != 2 or probs.shape != routing_map.shape:
        raise RuntimeError("routing_map_to_topk: routing_map and probs must both be [T, E]")
    rm = routing_map.contiguous()
    if rm.dtype == torch.bool:
        rm = rm.view(torch.uint8)
    elif rm.element_size() != 1:
        rm = (rm != 0).view(torch.uint8)
    probs = probs.contiguous()
    if probs.element_size() not in (2, 4):
        raise RuntimeError(f"routing_map_to_topk: unsupported probs dtype {probs.dtype}")
    dev = rm.device
    T, E = rm.shape
    stats = torch.empty((2,), dtype=torch.int32, device=dev)
    _hip.call("terrace_routing_map_count", _hip.ptr(rm), T, E, _hip.ptr(stats), _hip.stream(dev))
    mn, mx = stats.tolist()
    if T == 0:
        mn = mx = 0
    if mn != mx:
        raise RuntimeError("T-A2A requires exactly k experts per token (drop-less); observed per-row expert "
                           "counts differ")
    k = int(mn)
    if k == 0:
        raise RuntimeError("T-A2A got an all-empty routing_map (k=0); impossible under drop-less routing")
    expert_idx = torch.empty((T, k), dtype=torch.int64, device=dev)
    gates = torch.empty((T, k), dtype=probs.dtype, device=dev)
    _hip.call("terrace_routing_map_topk", _hip.ptr(rm), _hip.ptr(probs), probs.element_size(), T, E, k,
              _hip.ptr(expert_idx), _hip.ptr(gates), _hip.stream(dev))
    return expert_idx, gates


def hopa_send_splits(node_counts, world, rpn, my_local):
    """Hop-A counts-exchange send buffer (terrace/ta2a_dispatch.py:197-211 of the reference)."""
    _require()
    _hip.need_device(node_counts)
    node_counts = node_counts.contiguous()
    send = torch.empty((world,), dtype=torch.int64, device=node_counts.device)
    _hip.call("terrace_hopa_send_splits", _hip.ptr(node_counts), world, rpn, my_local, _hip.ptr(send),
              _hip.stream(node_counts.device))
    return send


# --------------------------------------------------------------------------------------
# torch.ops.terrace registration (reference schemas)
# --------------------------------------------------------------------------------------

_TORCH_LIB = None


def _register_torch_ops():
    global _TORCH_LIB
    if _TORCH_LIB is not None:
        return
    lib = torch.library.Library("terrace", "DEF")
    lib.define("passthrough(Tensor x) -> Tensor")
    lib.define("k1_arrival(Tensor rx, Tensor rslot, Tensor rgate, int quota, int epr, int rpn, int my_local) "
               "-> (Tensor, Tensor, Tensor, Tensor, Tensor)")
    lib.define("k2_pack(Tensor hidden, Tensor expert_idx, Tensor gates, int world, int n_experts, int rpn, "
               "int groups_m) -> (Tensor, Tensor, Tensor, Tensor, Tensor)")

    def _pass(x):
        _hip.need_device(x)
        xc = x.contiguous()
        y = torch.empty_like(xc)
        _hip.call("terrace_passthrough", _hip.ptr(xc), _hip.ptr(y), xc.numel() * xc.element_size(),
                  _hip.stream(x.device))
        return y

    def _k1(rx, rslot, rgate, quota, epr, rpn, my_local):
        return k1_arrival_raw(rx, rslot, rgate, quota, epr, rpn, my_local)

    def _k2(hidden, expert_idx, gates, world, n_experts, rpn, groups_m):
        return k2_pack_raw(hidden, expert_idx, gates, world, n_experts, rpn, groups_m)

    def _k1_meta(rx, rslot, rgate, quota, epr, rpn, my_local):
        P, H = rslot.shape[0] * quota, rx.shape[1]
        return (rx.new_empty((P, H)), rgate.new_empty((P,)), rslot.new_empty((P,)), rslot.new_empty((P,)),
                rslot.new_empty((rpn,)))

    def _k2_meta(hidden, expert_idx, gates, world, n_experts, rpn, groups_m):
        n_rows, q = expert_idx.shape[0] * groups_m, expert_idx.shape[1] // groups_m
        return (hidden.new_empty((n_rows, hidden.shape[1])), expert_idx.new_empty((n_rows, q)),
                gates.new_empty((n_rows, q)), expert_idx.new_empty((n_rows,)),
                expert_idx.new_empty((world // rpn,)))

    lib.impl("passthrough", _pass, "CUDA")
    lib.impl("k1_arrival", _k1, "CUDA")
    lib.impl("k2_pack", _k2, "CUDA")
    lib.impl("passthrough", lambda x: torch.empty_like(x), "Meta")
    lib.impl("k1_arrival", _k1_meta, "Meta")
    lib.impl("k2_pack", _k2_meta, "Meta")

    # A call through torch.ops on tensors that require grad must not drop the gradient silently: the two float
    # outputs of each operator hang on the same adjoints as the functional entry points.
    def _below_autograd(op, *args):
        with torch._C._AutoDispatchBelowAutograd():
            return op(*args)

    def _k1_autograd(rx, rslot, rgate, quota, epr, rpn, my_local):
        if not rx.is_cuda:
            return _below_autograd(torch.ops.terrace.k1_arrival, rx, rslot, rgate, quota, epr, rpn, my_local)
        return TerraceK1ArrivalFn.apply(rx, rslot, rgate, quota, epr, rpn, my_local)

    def _k2_autograd(hidden, expert_idx, gates, world, n_experts, rpn, groups_m):
        if not hidden.is_cuda:
            return _below_autograd(torch.ops.terrace.k2_pack, hidden, expert_idx, gates, world, n_experts, rpn,
                                   groups_m)
        return TerraceK2PackFn.apply(hidden, expert_idx, gates, world, n_experts, rpn, groups_m)

    lib.impl("k1_arrival", _k1_autograd, "Autograd")
    lib.impl("k2_pack", _k2_autograd, "Autograd")
    _TORCH_LIB = lib


# --------------------------------------------------------------------------------------
# autograd wrappers and functional entry points (reference names)
# --------------------------------------------------------------------------------------

class TerracePassthroughFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        return torch.ops.terrace.passthrough(x)

    @staticmethod
    def backward(ctx, grad_out):
        return grad_out


def passthrough(x: torch.Tensor) -> torch.Tensor:
    """Identity copy through the streaming-copy kernel: a new tensor, bit-equal to ``x``."""
    _require()
    return TerracePassthroughFn.apply(x)


def stream_probe(kind: str, x, y):
    """One launch of a stream probe (``read`` | ``write`` | ``sum8`` | ``copy``): ``y``'s byte size is what the
    probe writes (reads, for ``read``); ``sum8`` reads eight times that from ``x``.  Returns ``y``."""
    _require()
    _hip.need_device(x, y)
    code = {"read": _hip.PROBE_READ, "write": _hip.PROBE_WRITE, "sum8": _hip.PROBE_SUM8, "copy": _hip.PROBE_COPY}[kind]
    nbytes = y.numel() * y.element_size()
    need = {"read": nbytes, "write": 0, "sum8": 8 * nbytes, "copy": nbytes}[kind]
    if not y.is_contiguous() or (x is not None and (not x.is_contiguous() or x.numel() * x.element_size() < need)):
        raise RuntimeError("stream_probe: contiguous tensors, and a source at least as large as the probe reads")
    if x is None and need:
        raise RuntimeError(f"stream_probe: {kind} needs a source")
    _hip.call("terrace_stream_probe", code, _hip.ptr(x), _hip.ptr(y), nbytes, _hip.stream(y.device))
    return y


def _k1_grad_rx(g_send, pair_pos, rx_shape, quota):
    """Adjoint of ``send_buf = rx[r_idx]``: row r sums its quota pairs, in pair order."""
    return combine(g_send, pair_pos.view(rx_shape[0], quota), None, out_dtype=g_send.dtype)


def _k1_grad_rgate(g_gate, pair_pos, rgate_shape):
    """Adjoint of ``gate_pairs = rgate.flatten()[ordo]``: a permutation, so a plain gather."""
    return gather_rows(g_gate.reshape(-1, 1), pair_pos).view(rgate_shape)


class TerraceK1ArrivalFn(torch.autograd.Function):
    """Forward = the arrival kernel; backward = the two gather adjoints
    (terrace/ops/__init__.py:303-365 of the reference), also as kernels."""

    @staticmethod
    def forward(ctx, rx, rslot, rgate, quota, epr, rpn, my_local):
        send_buf, gate_pairs, r_idx, slot_idx, i_send, pair_pos = k1_arrival_raw(
            rx, rslot, rgate, quota, epr, rpn, my_local, want_pair_pos=True)
        ctx.save_for_backward(pair_pos)
        ctx.k1_geom = (quota, rx.shape, rgate.shape)
        ctx.mark_non_differentiable(r_idx, slot_idx, i_send)
        return send_buf, gate_pairs, r_idx, slot_idx, i_send

    @staticmethod
    def backward(ctx, g_send, g_gate, _g_r, _g_s, _g_i):
        (pair_pos,) = ctx.saved_tensors
        quota, rx_shape, rgate_shape = ctx.k1_geom
        grad_rx = grad_rgate = None
        if ctx.needs_input_grad[0] and g_send is not None:
            grad_rx = _k1_grad_rx(g_send.contiguous(), pair_pos, rx_shape, quota)
        if ctx.needs_input_grad[2] and g_gate is not None:
            grad_rgate = _k1_grad_rgate(g_gate.contiguous(), pair_pos, rgate_shape)
        return grad_rx, None, grad_rgate, None, None, None, None


def k1_arrival(rx, rslot, rgate, quota: int, epr: int, rpn: int, my_local: int = 0):
    """Arrival-side fused chain: (send_buf, gate_pairs, r_idx, slot_idx, i_send)."""
    _require()
    if rx.requires_grad or rgate.requires_grad:
        return TerraceK1ArrivalFn.apply(rx, rslot, rgate, quota, epr, rpn, my_local)
    return k1_arrival_raw(rx, rslot, rgate, quota, epr, rpn, my_local)


class _K1SendEdge(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rx, pair_pos, send_buf, quota):
        ctx.save_for_backward(pair_pos)
        ctx.geom = (rx.shape, quota)
        return send_buf

    @staticmethod
    def backward(ctx, g_send):
        (pair_pos,) = ctx.saved_tensors
        rx_shape, quota = ctx.geom
        g = _k1_grad_rx(g_send.contiguous(), pair_pos, rx_shape, quota) if ctx.needs_input_grad[0] else None
        return g, None, None, None


class _K1GateEdge(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rgate, pair_pos, gate_pairs):
        ctx.save_for_backward(pair_pos)
        ctx.geom = rgate.shape
        return gate_pairs

    @staticmethod
    def backward(ctx, g_gate):
        (pair_pos,) = ctx.saved_tensors
        g = _k1_grad_rgate(g_gate.contiguous(), pair_pos, ctx.geom) if ctx.needs_input_grad[0] else None
        return g, None, None


def k1_arrival_segment(rx, rslot, rgate, quota: int, epr: int, rpn: int, my_local: int = 0):
    """Same values as ``k1_arrival``; the two float outputs hang on separate autograd edges
    rooted at ``rx`` / ``rgate`` (terrace/ops/__init__.py:452-474 of the reference)."""
    with torch.no_grad():
        send_buf, gate_pairs, r_idx, slot_idx, i_send, pair_pos = k1_arrival_raw(
            rx.detach(), rslot, rgate.detach(), quota, epr, rpn, my_local, want_pair_pos=True)
    send_buf = _K1SendEdge.apply(rx, pair_pos, send_buf, quota)
    gate_pairs = _K1GateEdge.apply(rgate, pair_pos, gate_pairs)
    return send_buf, gate_pairs, r_idx, slot_idx, i_send


class TerraceK2PackFn(torch.autograd.Function):
    """Forward = the send-side kernels; backward = the adjoints of the two differentiable outputs
    (terrace/ops/k2_ref.py:77-81 of the reference: ``payload``, a deduplicated gather of ``hidden``, and
    ``gate_rows``, a permutation gather of ``gates``, carry gradients), also as kernels: a token sums the
    gradients of its M send rows in ascending row order, a gate takes the gradient of the one cell it was
    copied to."""

    @staticmethod
    def forward(ctx, hidden, expert_idx, gates, world, n_experts, rpn, groups_m):
        (payload, mask, gate_rows, u_src, node_counts), ex = k2_pack_raw(
            hidden, expert_idx, gates, world, n_experts, rpn, groups_m, extras=True)
        _guard_k2(ex["status"], expert_idx, world, rpn, groups_m)
        ctx.save_for_backward(ex["token_rows"], ex["pair_table"], ex["sort_order"])
        ctx.k2_dtypes = (hidden.dtype, gates.dtype)
        ctx.mark_non_differentiable(mask, u_src, node_counts)
        return payload, mask, gate_rows, u_src, node_counts

    @staticmethod
    def backward(ctx, g_payload, _g_mask, g_gate_rows, _g_src, _g_counts):
        token_rows, pair_table, sort_order = ctx.saved_tensors
        hidden_dtype, gates_dtype = ctx.k2_dtypes
        d_hidden = d_gates = None
        if ctx.needs_input_grad[0] and g_payload is not None:
            d_hidden = combine(g_payload.contiguous(), token_rows, None, out_dtype=hidden_dtype)
        if ctx.needs_input_grad[2] and g_gate_rows is not None:
            T, k = pair_table.shape
            by_rank = gather_rows(g_gate_rows.contiguous().to(gates_dtype).reshape(-1, 1), pair_table.reshape(-1))
            d_gates = torch.zeros((T, k), dtype=gates_dtype, device=pair_table.device)
            rows = torch.arange(T, device=pair_table.device, dtype=torch.int64).unsqueeze(1).expand(T, k)
            scatter_elems(by_rank, rows, sort_order, d_gates)
        return d_hidden, None, d_gates, None, None, None, None


def _guard_k2(status, expert_idx, world, rpn, groups_m):
    """The plan's guard (first call per shape and every 256th, one read-back when it fires) applied to the
    status words of a send-side call: an id out of range, a fan-out other than M or a node off the quota
    raise ValueError as in the reference (terrace/ta2a.py:161-204, terrace/ops/k2_ref.py:108)."""
    from .. import ta2a as _plan            # deferred: ta2a imports this module
    T, k = expert_idx.shape
    _plan._guard(status, T, k, world // rpn, groups_m)


def k2_pack(hidden, expert_idx, gates, world: int, n_experts: int, rpn: int, groups_m: int):
    """Send-side fused chain: (payload, mask, gate_rows, u_src, node_counts).  ``payload`` and ``gate_rows``
    carry gradients to ``hidden`` and ``gates``; a malformed routing raises ValueError on the guard's cadence."""
    _require()
    if torch.is_grad_enabled() and (hidden.requires_grad or gates.requires_grad):
        return TerraceK2PackFn.apply(hidden, expert_idx, gates, world, n_experts, rpn, groups_m)
    out, ex = k2_pack_raw(hidden, expert_idx, gates, world, n_experts, rpn, groups_m, extras=True)
    _guard_k2(ex["status"], expert_idx, world, rpn, groups_m)
    return out


def k1_arrival_ref(rx, rslot, rgate, quota: int, epr: int, rpn: int, my_local: int = 0):
    """The name under which the reference keeps the executable specification of K1
    (terrace/ops/__init__.py:255-300 there: the composed torch chain).  This build has one implementation of
    that specification, the kernels, so the name resolves to them: same arguments, same five outputs, same
    gradients as :func:`k1_arrival`."""
    if rslot.dim() == 2 and rslot.shape[1] != quota:
        raise AssertionError(f"rslot dim 1 {rslot.shape[1]} != quota {quota} (quota wire-format contract)")
    return k1_arrival(rx, rslot, rgate, quota, epr, rpn, my_local)


__all__ = [
    "OpsLoadError", "OpsState", "TerracePassthroughFn", "TerraceK1ArrivalFn", "TerraceK2PackFn",
    "custom_ops_enabled", "k1_arrival", "k1_arrival_ref", "k1_arrival_segment", "k2_pack", "passthrough", "reset",
    "status",
    "regroup", "combine", "gather_rows", "scatter_rows", "index_chain", "index_chain2", "hist", "argsort_small", "hopa_send_splits",
    "plan_general", "build_mask", "scatter_elems", "expand_mask", "arrival_pairs", "routing_map_topk", "segment_table", "pair_places",
    "wire_words", "k2_pack_wire", "k1_arrival_wire", "regroup_wire", "hopb_scatter", "hopb_scatter_move",
    "k1_arrival_static",
]
