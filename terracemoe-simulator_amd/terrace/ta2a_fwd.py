"""T-A2A forward primitives on MI355X, and the one-GPU loop-back forward.

Same names as the reference module (terrace/ta2a_fwd.py there) for the primitives the
dispatch/combine path is made of: ``fixed_hist``, ``_stable_argsort_small``,
``_pack_quota_wire``, ``_expand_arrival_quota``.  The reference's ``ta2a_moe_forward`` strings
them together around four all-to-all exchanges; on one GPU those exchanges cannot run, so
``ta2a_loopback_forward`` runs the same stages with the rank's own Hop-A send buffer looped
back as its arrival buffer (slot ids are node-local, so that is a well-formed arrival set of
the balanced size) and every expert slot of the node treated as local.
"""
from __future__ import annotations

import os
from ctypes import c_int64, c_void_p

import torch

from . import _hip, _planes
from . import ops as _ops


def fixed_hist(idx: torch.Tensor, n_buckets: int) -> torch.Tensor:
    """Fixed-length int64 histogram (``bincount(idx, minlength=n_buckets)`` without the sync).  An index outside
    ``[0, n_buckets)`` is counted nowhere (the reference's ``scatter_add_`` would fail on it); ``terrace.ops.hist``
    also returns the status words that report it."""
    out, _ = _ops.hist(idx, n_buckets)
    return out


def _stable_argsort_small(key: torch.Tensor, n_buckets: int) -> torch.Tensor:
    """Stable ascending argsort of a small-range integer key (a counting sort)."""
    order, _ = _ops.argsort_small(key, n_buckets)
    return order


def _pack_quota_wire(expert_idx, gates, inverse, payload, n_rows: int, slots: int, quota: int,
                     n_experts: int, *, sorted_rows: bool = False):
    """Quota Hop-A id/gate planes: ``[n_rows, quota]`` ascending node-local slot ids (int64)
    and the co-indexed gates in the payload's dtype.  ``sorted_rows`` is accepted for
    signature compatibility; the kernel ranks each row itself, which is the identity on an
    ascending row."""
    _ops._require()
    _hip.need_device(expert_idx, gates, inverse, payload)
    if gates.dtype != payload.dtype and payload.dtype != torch.uint8:
        raise RuntimeError(f"Index put requires the source and destination dtypes match, got {payload.dtype} "
                           f"for the destination and {gates.dtype} for the source.")
    expert_idx, gates, inverse = expert_idx.contiguous(), gates.contiguous(), inverse.contiguous()
    T, k = expert_idx.shape
    dev = expert_idx.device
    slot_tab = torch.zeros((n_rows, quota), dtype=torch.int64, device=dev)
    gate_tab = torch.zeros((n_rows, quota), dtype=gates.dtype, device=dev)
    st = _hip.new_status(dev)
    _hip.call("terrace_pack_quota_wire", _hip.ptr(expert_idx), _hip.ptr(gates), _hip.ptr(inverse), T, k,
              gates.element_size(), n_rows, slots, quota, _hip.ptr(slot_tab), _hip.ptr(gate_tab), _hip.ptr(st),
              _hip.stream(dev))
    return slot_tab, gate_tab


def _expand_arrival_quota(rslot: torch.Tensor):
    """(r_idx, slot_idx) pairs straight off the quota wire table, row-major."""
    R, quota = rslot.shape
    r_idx = torch.arange(R, device=rslot.device, dtype=torch.int64).unsqueeze(1).expand(R, quota).reshape(-1)
    return r_idx, rslot.reshape(-1)


def _expand_arrival(rmask: torch.Tensor, slots: int, quota):
    """Arrival-side (row, slot) demand pairs from shipped bitmasks, before the owner reorder.

    ``quota`` None: every set bit, row-major with columns ascending (a data-dependent count,
    read back from the device).  Otherwise exactly ``quota`` columns per row: its set columns
    ascending, then -- only for a row holding fewer -- its unset columns ascending, which is
    the order the reference's distinct-key top-k gives."""
    return _ops.expand_mask(rmask, slots, quota)


def build_expansion(expert_idx, inverse, n_rows: int, world: int, n_experts: int, rpn: int = 8,
                    groups_m: int | None = None, *, sorted_rows: bool = False, slot_flat=None):
    """Per-send-row int64 bitmask of the destination node's expert slots that want the token:
    bit j of row r is set iff node-local slot j is one of the token's experts.  Requires
    ``epr*rpn <= 63``.  ``groups_m`` / ``sorted_rows`` / ``slot_flat`` only select cheaper
    formulations in the reference and never change a bit; one kernel serves all of them."""
    slots = (n_experts // world) * rpn
    if slots > 63:
        raise ValueError(f"{slots} expert slots per node exceeds the int64 mask")
    mask, _ = _ops.build_mask(expert_idx, inverse, n_rows, slots)
    return mask


def general_hopa_planes(x, expert_idx, gates, world: int, n_experts: int, rpn: int = 8, token_rows_out=None):
    """Send side of the general (non-quota) branch: (payload, mask, gate_rows, u_src,
    node_counts, inverse, u_node) with ``mask`` the [n_rows] int64 bitmask plane and ``gate_rows``
    the sparse [n_rows, slots] plane in the payload dtype.

    The payload ``x[u_src]`` is moved as a scatter over the token -> send rows table (each token's row is read once
    and written to its rows) rather than as a gather that reads a token's row once per copy; a list passed as
    ``token_rows_out`` receives that [T, min(k, n_nodes)] table (-1 padded), which is also the second level of the
    combine."""
    from .ta2a import plan_ta2a
    slots = (n_experts // world) * rpn
    if gates.dtype != x.dtype:
        raise RuntimeError(f"Index put requires the source and destination dtypes match, got {x.dtype} "
                           f"for the destination and {gates.dtype} for the source.")
    u_src, u_node, node_counts, inverse = plan_ta2a(expert_idx, world, n_experts, rpn, groups_m=None)
    n_rows = u_src.numel()
    T, k = expert_idx.shape
    token_rows, _ = _ops.segment_table(u_src, T, min(k, world // rpn))
    if token_rows_out is not None:
        token_rows_out.append(token_rows)
    payload = _ops.scatter_rows(x, token_rows, n_rows)
    mask = build_expansion(expert_idx, inverse, n_rows, world, n_experts, rpn)
    gate_rows = torch.zeros((n_rows, slots), dtype=x.dtype, device=x.device)
    _ops.scatter_elems(gates, inverse, expert_idx, gate_rows, col_mod=slots)
    return payload, mask, gate_rows, u_src, node_counts, inverse, u_node


class LoopbackState(_planes.LazyFields):
    """What the combine needs from the dispatch, and what a caller may want to inspect: ``payload``, ``mask``,
    ``gate_rows``, ``u_src``, ``node_counts``, ``extras`` (dict), ``send_buf``, ``gate_pairs``, ``r_idx``,
    ``slot_idx``, ``i_send``, ``pair_pos``, ``permuted``, ``tokens_per_expert``, ``place`` ([P]: where each arrival row
    sits in the expert-order buffer, -1 = dropped), ``kept`` (None when drop-less) and ``capacity``.  The small planes
    live in one allocation and become tensors when first read."""


class OnePassState(_planes.LazyFields):
    """Dispatch state when Hop B ran as one pass (:func:`loopback_dispatch_onepass`): ``payload``, ``mask``,
    ``gate_rows``, ``u_src``, ``node_counts``, ``extras``, ``permuted``, ``tokens_per_expert``, ``place``, ``kept``,
    ``capacity``.  No arrival-order send buffer exists, so ``place`` is indexed by Hop-A pair ``row*quota + i``."""


_INDEX_STREAMS: dict = {}


def _index_stream(device) -> "torch.cuda.Stream":
    """The per-device stream (default priority) the index chain runs on beside the row movers."""
    key = torch.device(device).index
    if key is None:
        key = torch.cuda.current_device()
    s = _INDEX_STREAMS.get(key)
    if s is None:
        s = _INDEX_STREAMS[key] = torch.cuda.Stream(device=key)
    return s


def _adopt(stream, *items):
    """Tensors allocated under another stream that ``stream`` will also use: tell the allocator."""
    for t in items:
        if isinstance(t, dict):
            _adopt(stream, *t.values())
        elif isinstance(t, torch.Tensor) and t.is_cuda:
            t.record_stream(stream)


def loopback_dispatch(x, expert_idx, gates, world: int, n_experts: int, rpn: int = 8, groups_m: int = 1,
                      capacity: int | None = None, overlap: bool | None = None) -> LoopbackState:
    """Stages 2-4 on one GPU: index build + Hop-A pack, arrival chain, expert-order regroup.

    ``overlap`` (default: the ``TERRACE_OVERLAP`` environment switch, off unless "1"): every index plane
    of the three stages depends only on index planes of the stage before, never on moved rows -- the
    property the reference uses when it ships counts and metadata ahead of the payload
    (terrace/ta2a_dispatch.py:78-100, 399-412).  With ``overlap`` the whole index chain, the combine's
    place table included, runs ahead on a second stream while the current stream moves rows back to back,
    each mover waiting only for the event of its own stage's planes.  The results are the same tensors
    either way.  It is off by default because on one GPU it measured slower: the movers do run back to
    back, but each of the five cross-stream waits costs about 11 us where the index kernel it hides costs
    5 us (T=16384, H=7168 bf16: 1.81 ms a step against 1.69 ms).  The two-phase operators underneath are
    what a multi-GPU caller needs regardless, with the payload exchange between the phases."""
    epr = n_experts // world
    slots = epr * rpn
    k = expert_idx.shape[1]
    quota = k // groups_m
    if overlap is None:
        overlap = os.environ.get("TERRACE_OVERLAP", "0") == "1"
    if not overlap or x.shape[0] == 0:
        return _dispatch_one_slab(x, expert_idx, gates, world, n_experts, rpn, groups_m, capacity, onepass=False)

    _ops._check_k2(x, expert_idx, gates, world, n_experts, rpn, groups_m)
    dev = x.device
    rows = torch.cuda.current_stream(dev)
    index = _index_stream(dev)
    index.wait_stream(rows)
    with torch.cuda.stream(index):
        (mask, gate_rows, u_src, node_counts), extras = _ops.k2_pack_index(
            expert_idx, gates, world, n_experts, rpn, groups_m)
        packed = index.record_event()
        gate_pairs, r_idx, slot_idx, i_send, pair_pos, ws_arrival = _ops.k1_arrival_index(
            mask, gate_rows, quota, epr, rpn, 0)
        arrived = index.record_event()
        rg = _ops.regroup_index(slot_idx, slots, 0, capacity)
        regrouped = index.record_event()
        place = rg["dest"]
        where = _ops.index_chain2(place, pair_pos, extras["pair_table"])
        chained = index.record_event()
    _adopt(rows, mask, gate_rows, u_src, node_counts, extras, gate_pairs, r_idx, slot_idx, i_send, pair_pos,
           ws_arrival, rg, where)
    rows.wait_event(packed)
    payload = _ops.k2_pack_move(x, extras["workspace"], k, world, rpn, groups_m)
    rows.wait_event(arrived)
    send_buf = _ops.k1_arrival_move(payload, ws_arrival, quota, rpn)
    rows.wait_event(regrouped)
    permuted = _ops.regroup_move(send_buf, rg["workspace"], slots, capacity)
    rows.wait_event(chained)            # joins the index stream: nothing of it is in flight on return
    extras["where"] = where
    extras["kept_per_expert"] = rg["kept_per_expert"]
    return LoopbackState(None, (), payload=payload, mask=mask, gate_rows=gate_rows, u_src=u_src, node_counts=node_counts,
                         extras=extras, send_buf=send_buf, gate_pairs=gate_pairs, r_idx=r_idx, slot_idx=slot_idx,
                         i_send=i_send, pair_pos=pair_pos, permuted=permuted,
                         tokens_per_expert=rg["tokens_per_expert"], place=place, kept=rg["kept"], capacity=capacity)


def loopback_dispatch_onepass(x, expert_idx, gates, world: int, n_experts: int, rpn: int = 8, groups_m: int = 1,
                              capacity: int | None = None) -> OnePassState:
    """Stages 2-4 on one GPU with Hop B as ONE pass: index build + Hop-A pack, then every packed row written
    straight to the expert-order (capacity-padded) place of each of its pairs (``ops.hopb_scatter``).  Same
    ``permuted`` / ``tokens_per_expert`` as :func:`loopback_dispatch` and ``place == its place[its pair_pos]``;
    the arrival-order planes (send_buf, r_idx, slot_idx, i_send) are never formed."""
    return _dispatch_one_slab(x, expert_idx, gates, world, n_experts, rpn, groups_m, capacity, onepass=True)


_DISPATCH_LAYOUTS: dict = {}

# slab names of the planes terrace_dispatch addresses, in the order of enum terrace_dispatch_plane
_SLAB_NAME = {"u_node": "x.u_node", "inverse": "x.inverse", "node_offsets": "x.node_offsets",
              "pair_table": "x.pair_table", "sort_order": "x.sort_order", "token_rows": "x.token_rows",
              "gate_sorted": "x.gate_sorted", "pair_src": "x.pair_src", "where": "x.where", "status": "x.status",
              "status_hopb": "_status_b", "status_regroup": "_status_r", "order": "_order",
              "kept_per_expert": "x.kept_per_expert"}


def _align256(n):
    return (int(n) + 255) // 256 * 256


def _dispatch_layout(T, k, world, n_experts, rpn, groups_m, capacity, gdt, onepass):
    """The slab arrangement of a dispatch's small planes (cached per geometry) and, as ``lay.offsets``, the table
    of plane offsets ``terrace_dispatch`` takes.  Names: state fields as they are, ``x.<key>`` the entries of
    ``extras``, ``_<name>`` scratch nobody reads."""
    key = (T, k, world, n_experts, rpn, groups_m, capacity, gdt, onepass)
    lay = _DISPATCH_LAYOUTS.get(key)
    if lay is not None:
        return lay
    n_nodes, slots = world // rpn, (n_experts // world) * rpn
    S, P, quota = T * groups_m, T * k, k // groups_m
    cap = -1 if capacity is None else int(capacity)
    i64, i32, u8 = torch.int64, torch.int32, torch.uint8
    planes = [("mask", (S, quota), i64), ("gate_rows", (S, quota), gdt), ("u_src", (S,), i64),
              ("node_counts", (n_nodes,), i64), ("tokens_per_expert", (slots,), i64), ("place", (P,), i64),
              ("kept", (P,) if capacity is not None else None, torch.bool),
              ("x.u_node", (S,), i64), ("x.inverse", (P,), i64), ("x.node_offsets", (n_nodes,), i64),
              ("x.pair_table", (T, k), i64), ("x.sort_order", (T, k), i64), ("x.token_rows", (T, groups_m), i64),
              ("x.gate_sorted", (T, k), gdt), ("x.pair_src", (P,), i64), ("x.where", (T, k), i64),
              ("x.status", (4,), i32), ("x.kept_per_expert", (slots,), i64), ("_status_b", (4,), i32),
              ("_ws", (_hip.query("terrace_dispatch_workspace", T, k, world, n_experts, rpn, groups_m, cap,
                                  1 if onepass else 0),), u8)]
    if not onepass:
        planes += [("gate_pairs", (P,), gdt), ("r_idx", (P,), i64), ("slot_idx", (P,), i64), ("i_send", (rpn,), i64),
                   ("pair_pos", (P,), i64), ("_status_r", (4,), i32)]     # `order` is optional and nobody reads it here
    if len(_DISPATCH_LAYOUTS) > 64:
        _DISPATCH_LAYOUTS.clear()
    lay = _DISPATCH_LAYOUTS[key] = _planes.Layout(planes)
    lay.offsets = (c_int64 * len(_hip.DISPATCH_PLANES))(
        *[lay.at[n][0] if n in lay.at else -1 for n in (_SLAB_NAME.get(p, p) for p in _hip.DISPATCH_PLANES)])
    return lay


def _dispatch_one_slab(x, expert_idx, gates, world, n_experts, rpn, groups_m, capacity, onepass, stagewise=False):
    """Stages 2-4 through the C ABI with every small plane in one allocation: one library call
    (``terrace_dispatch``), or -- ``stagewise`` -- the three stage entry points one after the other (two with Hop B
    as one pass), which launch the same kernels on the same planes.  The combine's [T, k] place table is filled on
    the way: every Hop-A pair carries the entry it answers (pair_src) through the sorts, and the last one writes
    the pair's place there."""
    _ops._require()
    _hip.need_device(x, expert_idx, gates)
    _ops._check_k2(x, expert_idx, gates, world, n_experts, rpn, groups_m)
    x, expert_idx, gates = _hip.as_rows(x), expert_idx.contiguous(), gates.contiguous()
    dev = x.device
    T, k = expert_idx.shape
    epr, n_nodes = n_experts // world, world // rpn
    slots, quota = epr * rpn, k // groups_m
    S, P = T * groups_m, T * k
    cap = -1 if capacity is None else int(capacity)
    places = P if capacity is None else slots * cap
    row_bytes, gb = _hip.row_arg(x), gates.element_size()        # rows on a pitch keep it through every stage
    lay = _dispatch_layout(T, k, world, n_experts, rpn, groups_m, capacity, gates.dtype, onepass)
    slab = _planes.Slab(lay, dev)
    payload = _hip.empty_rows(S, x)
    permuted = _hip.empty_rows(places, x)
    send_buf = None if onepass else _hip.empty_rows(P, x)
    ptr, at, stream = _hip.ptr, slab.ptr, _hip.stream(dev)
    # the plan's guard (terrace/ta2a.py:161-204 of the reference): the status words are read back on the first
    # dispatch of a shape and on every 256th, after the last launch so the read-back waits for nothing extra
    from . import ta2a as _plan
    guard_key = (T, k, n_nodes, groups_m)
    guard = _plan._guard_due(guard_key)
    if not stagewise:
        _hip.call("terrace_dispatch", ptr(x), ptr(expert_idx), ptr(gates), T, row_bytes, gb, k, world, n_experts, rpn,
                  groups_m, cap, 1 if onepass else 0, ptr(payload), ptr(send_buf), ptr(permuted), c_void_p(slab.base),
                  lay.offsets, at("_ws"), slab.nbytes("_ws"), stream)
    else:
        ws = slab.base + lay.at["_ws"][0]
        n_k2 = _align256(_hip.query("terrace_k2_pack_workspace", T, k, n_nodes, groups_m))
        _hip.call("terrace_k2_pack", ptr(x), ptr(expert_idx), ptr(gates), T, row_bytes, gb, k, world, n_experts, rpn,
                  groups_m, ptr(payload), at("mask"), at("gate_rows"), at("u_src"), at("node_counts"), at("x.u_node"),
                  at("x.inverse"), at("x.node_offsets"), at("x.pair_table"), at("x.sort_order"), at("x.token_rows"),
                  at("x.gate_sorted"), at("x.pair_src"), at("x.where"), at("x.status"), c_void_p(ws), n_k2, stream)
        if onepass:
            _hip.call("terrace_hopb_scatter", ptr(payload), at("mask"), None, S, row_bytes, gb, quota, 0, slots, cap,
                      ptr(permuted), None, at("place"), at("kept"), None, at("tokens_per_expert"),
                      at("x.kept_per_expert"), at("x.pair_src"), at("x.where"), P, at("_status_b"), c_void_p(ws + n_k2),
                      slab.nbytes("_ws") - n_k2, stream)
        else:
            n_a = _align256(_hip.query("terrace_k1_arrival_workspace", S, quota, rpn))
            n_r = _align256(_hip.query("terrace_regroup_workspace", P, slots, cap))
            carried = c_void_p(ws + n_k2 + n_a + n_r)
            _hip.call("terrace_k1_arrival", ptr(payload), at("mask"), at("gate_rows"), S, row_bytes, gb, quota, epr,
                      rpn, 0, ptr(send_buf), at("gate_pairs"), at("r_idx"), at("slot_idx"), at("i_send"),
                      at("pair_pos"), at("x.pair_src"), carried, at("_status_b"), c_void_p(ws + n_k2), n_a, stream)
            _hip.call("terrace_regroup", ptr(send_buf), at("slot_idx"), None, P, row_bytes, gb, slots, 0, cap,
                      ptr(permuted), None, at("_order"), at("place"), at("kept"), at("tokens_per_expert"),
                      at("x.kept_per_expert"), carried, at("x.where"), P, at("_status_r"), c_void_p(ws + n_k2 + n_a),
                      n_r, stream)
    extras = _planes.LazyDict(slab, "x.")
    if guard:
        _plan._raise_from_status(extras["status"], T, k, groups_m)
        _plan._VERIFIED.add(guard_key)
    if onepass:
        return OnePassState(slab, ("kept",), payload=payload, permuted=permuted, extras=extras, capacity=capacity)
    return LoopbackState(slab, ("kept",), payload=payload, send_buf=send_buf, permuted=permuted, extras=extras,
                         capacity=capacity)


def _regroup_with_place(node_rx, my_slot, epr, my_local: int = 0, my_gate=None, tags=None, table=None):
    """Drop-less regroup that also returns each input row's place (the inverse of ``order``):
    (permuted, order, tokens_per_expert, place[, permuted_gate]).  ``tags`` / ``table`` as in ``ops.regroup``."""
    _ops._require()
    node_rx, my_slot = node_rx.contiguous(), my_slot.contiguous().reshape(-1)
    dev = my_slot.device
    P, H = node_rx.shape
    permuted = torch.empty_like(node_rx)
    order = torch.empty((P,), dtype=torch.int64, device=dev)
    place = torch.empty((P,), dtype=torch.int64, device=dev)
    tpe = torch.empty((epr,), dtype=torch.int64, device=dev)
    pgate, gate_bytes = None, 4
    if my_gate is not None:
        my_gate = my_gate.contiguous().reshape(-1)
        gate_bytes = my_gate.element_size()
        pgate = torch.empty((P,), dtype=my_gate.dtype, device=dev)
    n_tags = 0
    if tags is not None:
        tags, table = _ops._tag_plane(tags, P, dev), _ops._table_plane(table)
        n_tags = table.numel()
    st = _hip.new_status(dev)
    ws = _hip.workspace(_hip.query("terrace_regroup_workspace", P, epr, -1), dev)
    _hip.call("terrace_regroup", _hip.ptr(node_rx), _hip.ptr(my_slot), _hip.ptr(my_gate), P,
              H * node_rx.element_size(), gate_bytes, epr, my_local, -1, _hip.ptr(permuted), _hip.ptr(pgate),
              _hip.ptr(order), _hip.ptr(place), None, _hip.ptr(tpe), None, _hip.ptr(tags), _hip.ptr(table), n_tags,
              _hip.ptr(st), _hip.ptr(ws), ws.numel(), _hip.stream(dev))
    out = (permuted, order, tpe, place)
    return out + (pgate,) if my_gate is not None else out


def loopback_combine(ye, st, out_dtype=None, fp8_hidden=None, weights=None):
    """Stage 5, fused: ``y[t] = sum_s gate[t,s] * ye[place of (t, s-th smallest expert)]``.

    The k rows of a token are added in ascending expert id -- slot ascending inside a send row,
    node ascending across the token's rows -- which is the order the reference's two
    ``index_add`` levels add in (terrace/ta2a_fwd.py:661-670 there), accumulated in fp32.
    """
    where = st.extras.get("where")
    if where is None:
        if isinstance(st, OnePassState):
            where = _ops.index_chain(st.place, st.extras["pair_table"])
        else:
            where = _ops.index_chain2(st.place, st.pair_pos, st.extras["pair_table"])
    w = st.extras["gate_sorted"] if weights is None else weights
    return _ops.combine(ye, where, w, out_dtype=out_dtype, fp8_hidden=fp8_hidden)


def twolevel_combine(ye, st: LoopbackState, out_dtype=None):
    """Stage 5 in the reference's two levels (what a multi-GPU run would execute either side
    of the return exchanges): un-permute, per-row gate-weighted sum over the quota pairs, then
    per-token sum over the M rows.  Each level rounds to the payload dtype, as the reference."""
    R, q = st.mask.shape
    ret_place = _ops.index_chain(st.place, st.pair_pos).view(R, q)      # ye row of pair (r, i)
    red = _ops.combine(ye, ret_place, st.gate_rows, out_dtype=out_dtype)
    return _ops.combine(red, st.extras["token_rows"], None, out_dtype=out_dtype)


def ta2a_loopback_forward(x, expert_idx, gates, expert_fn, world: int, n_experts: int, rpn: int = 8,
                          groups_m: int = 1, capacity: int | None = None, onepass: bool = False):
    """dispatch -> ``expert_fn(permuted, tokens_per_expert) -> ye`` -> combine, on one GPU.  ``onepass`` runs
    Hop B as one scatter (same ``permuted``, no arrival-order planes in the returned state)."""
    dispatch = loopback_dispatch_onepass if onepass else loopback_dispatch
    st = dispatch(x, expert_idx, gates, world, n_experts, rpn, groups_m, capacity)
    ye = expert_fn(st.permuted, st.tokens_per_expert)
    return loopback_combine(ye, st), st


def ta2a_moe_forward(*_args, **_kwargs):
    raise NotImplementedError("ta2a_moe_forward needs the all-to-all exchanges of a multi-GPU run; this "
                              "one-GPU build provides ta2a_loopback_forward and the per-stage operators")
