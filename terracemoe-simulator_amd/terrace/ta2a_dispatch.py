"""T-A2A as the two halves of a token dispatcher, on one MI355X.

Same surface as the reference module (terrace/ta2a_dispatch.py there): ``routing_map_to_topk``,
``TA2AState``, ``ta2a_permute`` and ``ta2a_unpermute`` with the vendor's expert compute between
them.  The dispatch half returns (rows in local-expert order, rows per local expert, the
per-row gates, state); the gate is NOT multiplied here (the expert layer does that), and the
combine half adds each returned row once per (row, slot) pair and once per (token, node).
Both halves are differentiable: the float outputs hang on autograd edges whose backward passes
are the adjoint row movers (a fixed-fan gather-reduce for ``hidden_states``, an element gather
for ``probs``, a fan-k row scatter for ``expert_out``), so the router learns through
``permuted_probs`` as it does in the reference.

The reference runs four all-to-all exchanges inside these halves.  One GPU has no peers, so
the exchanges are loop-back: the rank's own Hop-A send buffer is its arrival buffer and every
Hop-B row stays on this card (pass ``intra_group=None``; a process group raises).  Slot ids
are node-local, so the looped-back rows form a well-formed arrival set of the balanced size;
all ``epr*rpn`` slots of the node then count as local experts, which makes
``tokens_per_expert`` ``[epr*rpn]`` long instead of ``[epr]``.  The wire containers are still
packed and unpacked around each (absent) exchange exactly where the reference does, under the
same ``TERRACE_TA2A_PACK`` mode switch.
"""
from __future__ import annotations

import os

import torch

from . import _hip
from . import ops as _ops
from . import ta2a as _plan
from . import ta2a_pack as _pk
from .ta2a_fwd import _expand_arrival, _regroup_with_place, general_hopa_planes


class TA2AState:
    """Intermediates handed from the dispatch half to the combine half; one per layer per
    microbatch, owned by the caller (terrace/ta2a_dispatch.py:62-74 of the reference)."""

    __slots__ = ("u_src", "r_idx", "order", "R", "T", "hidden",
                 "send_l", "recv_l", "is_l", "ir_l", "intra", "inter", "dtype",
                 "red_table", "tok_table", "where", "token_of_place")


def routing_map_to_topk(routing_map: torch.Tensor, probs: torch.Tensor):
    """[T, E] boolean map + [T, E] probabilities -> [T, k] expert ids (ascending per row) and
    their gates.  Requires exactly k set entries in every row and raises RuntimeError otherwise;
    one host synchronisation (the min and max of the per-row counts)."""
    return _ops.routing_map_topk(routing_map, probs)


class _PermutedEdge(torch.autograd.Function):
    """permuted[i] = hidden[token_of_place[i]]; adjoint: a token sums the k places it was copied to."""

    @staticmethod
    def forward(ctx, hidden_states, where, permuted):
        ctx.save_for_backward(where)
        ctx.dtype = hidden_states.dtype
        return permuted

    @staticmethod
    def backward(ctx, g):
        (where,) = ctx.saved_tensors
        return _ops.combine(g.contiguous(), where, None, out_dtype=ctx.dtype), None, None


class _ProbsEdge(torch.autograd.Function):
    """permuted_probs[where[t, j]] = probs[t, expert_idx[t, j]]; adjoint: the same two look-ups backwards."""

    @staticmethod
    def forward(ctx, probs, where, expert_idx, pprobs):
        ctx.save_for_backward(where, expert_idx)
        ctx.shape, ctx.dtype = probs.shape, probs.dtype
        return pprobs

    @staticmethod
    def backward(ctx, g):
        where, expert_idx = ctx.saved_tensors
        T, k = expert_idx.shape
        d_gates = _ops.gather_rows(g.contiguous().to(ctx.dtype).reshape(-1, 1), where.reshape(-1))
        d_probs = torch.zeros(ctx.shape, dtype=ctx.dtype, device=g.device)
        rows = torch.arange(T, device=g.device, dtype=torch.int64).unsqueeze(1).expand(T, k)
        _ops.scatter_elems(d_gates, rows, expert_idx, d_probs)
        return d_probs, None, None, None


class _UnpermuteFn(torch.autograd.Function):
    """y[t] = sum_j expert_out[where[t, j]] (two levels); adjoint: place where[t, j] receives dy[t]."""

    @staticmethod
    def forward(ctx, expert_out, red_table, tok_table, where, out_dtype):
        ctx.save_for_backward(where)
        ctx.n_places, ctx.dtype = expert_out.shape[0], expert_out.dtype
        return _ops.combine_two_level(expert_out, red_table, tok_table, out_dtype=out_dtype)

    @staticmethod
    def backward(ctx, gy):
        (where,) = ctx.saved_tensors
        return _ops.scatter_rows(gy.contiguous().to(ctx.dtype), where, ctx.n_places), None, None, None, None


def _loopback_only(*groups):
    for g in groups:
        if g is not None:
            raise NotImplementedError("this one-GPU build runs the exchanges loop-back; pass intra_group=None "
                                      "and inter_group=None")


def ta2a_permute(hidden_states, probs, routing_map, *, world, rank, rpn, n_experts, intra_group=None,
                 inter_group=None, groups_m=None):
    """Dispatch half: (permuted [P,H], tokens_per_expert, permuted_probs [P], state)."""
    _loopback_only(intra_group, inter_group)
    _ops._require()
    _hip.need_device(hidden_states, probs, routing_map)
    epr = n_experts // world
    slots = epr * rpn
    n_nodes = world // rpn
    my_local = rank % rpn
    pack_mode = _pk.pack_mode()
    hidden_states = hidden_states.contiguous()

    expert_idx, gates = routing_map_to_topk(routing_map, probs)
    T, k = expert_idx.shape
    if groups_m:
        assert k % groups_m == 0, f"k={k} not divisible by groups_m={groups_m}"
    quota = (k // groups_m) if groups_m else None

    # Quota branch under the default "small" container mode: the three stage kernels write and read the
    # wire containers themselves, so no pack / unpack pass runs at all.
    fused_wire = quota is not None and pack_mode == "small"
    if quota is not None:
        if gates.dtype != hidden_states.dtype:
            raise RuntimeError(f"Index put requires the source and destination dtypes match, got "
                               f"{hidden_states.dtype} for the destination and {gates.dtype} for the source.")
        packer = _ops.k2_pack_wire if fused_wire else (lambda *a: _ops.k2_pack_raw(*a, extras=True))
        (payload, mask, gate_rows, u_src, node_counts), ex = packer(
            hidden_states, expert_idx, gates, world, n_experts, rpn, groups_m)
        _plan._guard(ex["status"], T, k, n_nodes, groups_m)
        u_node = ex["u_node"]
    else:
        token_rows = []
        payload, mask, gate_rows, u_src, node_counts, _inverse, u_node = general_hopa_planes(
            hidden_states, expert_idx, gates, world, n_experts, rpn, token_rows_out=token_rows)

    # Hop A (loop-back): what was packed for the wire is what arrives
    if fused_wire:
        rx, rwire = payload, ex["wire"]
    elif pack_mode == "small":
        sbuf, lay = _pk.hopa_pack_small(gate_rows, mask)
        rgate, rmask = _pk.hopa_unpack_small(sbuf, lay)
        _pk.assert_not_aliased(sbuf, rgate, rmask)
        rx = payload
    elif pack_mode == "full":
        sbuf, lay = _pk.hopa_pack(payload, gate_rows, mask)
        rx, rgate, rmask = _pk.hopa_unpack(sbuf, lay)
        _pk.assert_not_aliased(sbuf, rx, rgate, rmask)
    else:
        rx, rmask, rgate = payload, mask, gate_rows
    R = rx.shape[0]

    if fused_wire:
        # Hop B (loop-back): the container the arrival kernel wrote is what the expert card reads
        node_rx, my_meta, r_idx, _i_send, pair_pos, my_slot = _ops.k1_arrival_wire(
            rx, rwire, gates.dtype, quota, epr, rpn, my_local, want_slot_idx=True)   # = my_meta[:, 0], dense
        permuted, order, tokens_per_expert, place, pprobs = _ops.regroup_wire(node_rx, my_meta, gates.dtype, slots, 0)
    else:
        if quota is not None:
            exp_rx, gate_pairs, r_idx, slot_idx, _i_send, pair_pos = _ops.k1_arrival_raw(
                rx, rmask, rgate, quota, epr, rpn, my_local, want_pair_pos=True)
        else:
            r_in, s_in = _expand_arrival(rmask, slots, None)
            # index planes first, then the rows as a scatter over the per-row table of arrival positions (which the
            # combine's first level needs anyway): each arrived row is read once, not once per pair
            _none, gate_pairs, r_idx, slot_idx, _i_send, _ordo = _ops.arrival_pairs(rx, r_in, s_in, rgate, epr, rpn,
                                                                                   move=False)
            per_row, _ = _ops.segment_table(r_idx, R, min(k, slots))
            exp_rx = _ops.scatter_rows(rx, per_row, r_idx.numel())
        # Hop B (loop-back)
        node_rx = exp_rx
        if pack_mode != "off":
            bbuf = _pk.hopb_pack_meta(slot_idx, gate_pairs)
            my_slot, my_gate = _pk.hopb_unpack_meta(bbuf, gate_pairs.dtype)
        else:
            my_slot, my_gate = slot_idx, gate_pairs
        # every slot of the node is local under loop-back
        permuted, order, tokens_per_expert, place, pprobs = _regroup_with_place(node_rx, my_slot, slots, 0, my_gate)

    st = TA2AState()
    st.u_src, st.r_idx, st.order = u_src, r_idx, order
    st.R, st.T, st.hidden = R, T, hidden_states.shape[1]
    st.send_l = st.recv_l = st.is_l = st.ir_l = None
    st.intra, st.inter, st.dtype = intra_group, inter_group, hidden_states.dtype
    if quota is not None:
        st.red_table = _ops.index_chain(place, pair_pos).view(R, quota)
        st.tok_table = ex["token_rows"]
    else:
        st.red_table = _ops.index_chain(place, per_row)
        st.tok_table = token_rows[0]
    st.where, st.token_of_place = _ops.pair_places(order, r_idx, my_slot, u_src, u_node, expert_idx, slots)
    if torch.is_grad_enabled():
        if hidden_states.requires_grad:
            permuted = _PermutedEdge.apply(hidden_states, st.where, permuted)
        if probs.requires_grad:
            pprobs = _ProbsEdge.apply(probs, st.where, expert_idx, pprobs)
    return permuted, tokens_per_expert, pprobs, st


def ta2a_unpermute(expert_out, st: TA2AState, out_like):
    """Combine half: send expert outputs back to their tokens along the reverse of the dispatch.

    No gate multiply (the expert layer already applied ``permuted_probs``).  Two levels, as the
    reference: a send row sums the outputs of its (row, slot) pairs in arrival order, a token sums
    its rows in ascending row order; each level accumulates in fp32 and rounds once to the
    tensor dtype."""
    _hip.need_device(expert_out)
    if torch.is_grad_enabled() and expert_out.requires_grad:
        return _UnpermuteFn.apply(expert_out, st.red_table, st.tok_table, st.where, out_like.dtype)
    # loop-back: no exchange stands between the two levels, so one pass computes both (same bits, and the [R, H]
    # plane of per-row sums never reaches memory)
    return _ops.combine_two_level(expert_out, st.red_table, st.tok_table, out_dtype=out_like.dtype)


# --------------------------------------------------------------------------------------
# The overlap seam: the same two halves cut into the segments a hand-written layer backward replays
# (terrace/ta2a_dispatch.py:500-1013 of the reference)
# --------------------------------------------------------------------------------------
# The vendor layer this seam plugs into is one autograd.Function with a hand-written backward: the forward is cut
# into independent sub-graphs whose inputs are detached leaves, the exchange between two sub-graphs sits outside
# autograd, and the backward unpacks ``save_tensors`` by FIXED POSITION and replays the exchange by hand.  The
# dispatch half therefore appends exactly seven entries and the combine half three, in this order:
#   0 payload          graph rooted at hidden_states      (permute1_graph)
#   1 gate_rows        graph rooted at probs              (permuted_probs_graph)
#   2 None                                                  (num_global_tokens_per_local_expert_cpu)
#   3 rx_d             detached leaf: what Hop A delivered (permute2_input_detach)
#   4 permuted         graph rooted at rx_d               (permute2_graph)
#   5 rgate_d          detached leaf                       (permute2_prob_detach)
#   6 permuted_probs   graph rooted at rgate_d            (permute2_prob_graph)
#   7 eo_d             detached leaf: the expert output    (unpermute1_input_detach)
#   8 red              graph rooted at eo_d               (unpermute1_graph)
#   9 back_d           detached leaf: what Hop A returned  (unpermute2_input_detach)
# and the returned y is a graph rooted at back_d.  On one GPU both exchanges are loop-back, so the leaf at a
# segment boundary holds the very rows the previous segment produced; every sub-graph's backward is one of the
# row movers (a fixed-fan gather-reduce, a fan-out row scatter, an element gather or scatter).

_ENV_SHARED_OVERLAP = "TERRACE_SHARED_OVERLAP"
_SHARED_OVERLAP: bool | None = None


def shared_overlap_enabled() -> bool:
    """Where the shared-expert callback runs inside the dispatch half: after Hop A has been launched (default), or
    -- ``TERRACE_SHARED_OVERLAP=0`` -- after every dispatch exchange.  Same operators and operands either way.
    Read once and cached (terrace/ta2a_dispatch.py:604-621 of the reference)."""
    global _SHARED_OVERLAP
    if _SHARED_OVERLAP is None:
        _SHARED_OVERLAP = os.environ.get(_ENV_SHARED_OVERLAP, "1").strip() != "0"
    return _SHARED_OVERLAP


def reset_shared_overlap() -> None:
    """Forget the cached switch (test hook)."""
    global _SHARED_OVERLAP
    _SHARED_OVERLAP = None


def ta2a_enabled(ep_world: int, rpn: int = 8) -> bool:
    """Whether T-A2A applies: switched on (``TERRACE_TA2A=1``) and the expert-parallel group spans at least two
    nodes -- with one node there is no fabric hop to deduplicate (terrace/ta2a_dispatch.py:1016-1020)."""
    if os.environ.get("TERRACE_TA2A") != "1":
        return False
    return ep_world // rpn >= 2


class _TopkGatesEdge(torch.autograd.Function):
    """gates[t, j] = probs[t, expert_idx[t, j]]; adjoint: scatter back to the chosen entries."""

    @staticmethod
    def forward(ctx, probs, expert_idx, gates):
        ctx.save_for_backward(expert_idx)
        ctx.shape, ctx.dtype = probs.shape, probs.dtype
        return gates.view_as(gates)

    @staticmethod
    def backward(ctx, g):
        (expert_idx,) = ctx.saved_tensors
        T, k = expert_idx.shape
        d_probs = torch.zeros(ctx.shape, dtype=ctx.dtype, device=g.device)
        rows = torch.arange(T, device=g.device, dtype=torch.int64).unsqueeze(1).expand(T, k)
        _ops.scatter_elems(g.contiguous().to(ctx.dtype), rows, expert_idx, d_probs)
        return d_probs, None, None


class _GatherReduceEdge(torch.autograd.Function):
    """out[i] = sum_j src[table[i, j]] (entries < 0 contribute nothing), computed by the caller; adjoint: row
    table[i, j] of the source receives g[i]."""

    @staticmethod
    def forward(ctx, src, table, out):
        ctx.save_for_backward(table)
        ctx.n_src, ctx.dtype = src.shape[0], src.dtype
        return out.view_as(out)

    @staticmethod
    def backward(ctx, g):
        (table,) = ctx.saved_tensors
        return _ops.scatter_rows(g.contiguous().to(ctx.dtype), table, ctx.n_src), None, None


class _FanOutEdge(torch.autograd.Function):
    """out[table[r, j]] = src[r] for every entry >= 0, computed by the caller; adjoint: a source row sums the
    gradients of its copies in table order."""

    @staticmethod
    def forward(ctx, src, table, out):
        ctx.save_for_backward(table)
        ctx.dtype = src.dtype
        return out.view_as(out)

    @staticmethod
    def backward(ctx, g):
        (table,) = ctx.saved_tensors
        return _ops.combine(g.contiguous(), table, None, out_dtype=ctx.dtype), None, None


class _GateCellsEdge(torch.autograd.Function):
    """pprobs[table[r, j]] = rgate[r, cols[r, j]] for every entry >= 0, computed by the caller; adjoint: the cell
    takes the gradient of the one place it was copied to."""

    @staticmethod
    def forward(ctx, rgate, table, cols, pprobs):
        ctx.save_for_backward(table, cols)
        ctx.shape, ctx.dtype = rgate.shape, rgate.dtype
        return pprobs.view_as(pprobs)

    @staticmethod
    def backward(ctx, g):
        table, cols = ctx.saved_tensors
        R, w = table.shape
        vals = _ops.gather_rows(g.contiguous().to(ctx.dtype).reshape(-1, 1), table.reshape(-1))
        d = torch.zeros(ctx.shape, dtype=ctx.dtype, device=g.device)
        rows = torch.arange(R, device=g.device, dtype=torch.int64).unsqueeze(1).expand(R, w)
        _ops.scatter_elems(vals, rows, cols, d)          # padding entries carry column -1 and are skipped
        return d, None, None, None


class _SparseGateRowsEdge(torch.autograd.Function):
    """General branch: gate_rows[inverse[t*k+j], expert_idx[t, j] % slots] = gates[t, j]; adjoint: the gather."""

    @staticmethod
    def forward(ctx, gates, cells, gate_rows):
        ctx.save_for_backward(cells)
        ctx.shape, ctx.dtype = gates.shape, gates.dtype
        return gate_rows.view_as(gate_rows)

    @staticmethod
    def backward(ctx, g):
        (cells,) = ctx.saved_tensors
        return _ops.gather_rows(g.contiguous().to(ctx.dtype).reshape(-1, 1), cells).view(ctx.shape), None, None


def ta2a_permute_overlap(hidden_states, probs, routing_map, *, world, rank, rpn, n_experts, intra_group=None,
                         inter_group=None, groups_m=None, save_tensors, run_shared_experts=None):
    """Dispatch half of the overlap seam: the math of :func:`ta2a_permute`, cut at the points the vendor layer's
    hand-written backward expects (see the seat list above).

    Returns (permuted, tokens_per_expert, permuted_probs, share_experts_output, state).  ``run_shared_experts`` is
    called once, with no arguments, after Hop A would have been launched (or after every dispatch exchange with
    ``TERRACE_SHARED_OVERLAP=0``)."""
    _loopback_only(intra_group, inter_group)
    _ops._require()
    _hip.need_device(hidden_states, probs, routing_map)
    epr = n_experts // world
    slots = epr * rpn
    n_nodes = world // rpn
    my_local = rank % rpn
    H = hidden_states.shape[-1]
    pack_mode = _pk.pack_mode()
    overlap_shared = shared_overlap_enabled()
    share_experts_output = None
    shared_now = (lambda: run_shared_experts()) if run_shared_experts is not None else (lambda: None)

    with torch.enable_grad():
        # ---- segment 1: routing planes, plan, Hop-A send buffers (graphs rooted at hidden_states / probs)
        expert_idx, gates = routing_map_to_topk(routing_map, probs)
        T, k = expert_idx.shape
        if probs.requires_grad:
            gates = _TopkGatesEdge.apply(probs, expert_idx, gates)
        h = hidden_states.reshape(-1, H)
        gates_p = gates.to(h.dtype)              # the gate plane rounds where the payload's dtype says
        if groups_m:
            assert k % groups_m == 0, f"k={k} not divisible by groups_m={groups_m}"
        quota = (k // groups_m) if groups_m else None
        if quota is not None:
            (payload, mask, gate_rows, u_src, node_counts), ex = _ops.k2_pack_raw(
                h.detach(), expert_idx, gates_p.detach(), world, n_experts, rpn, groups_m, extras=True)
            _plan._guard(ex["status"], T, k, n_nodes, groups_m)
            u_node, tok_table = ex["u_node"], ex["token_rows"]
            if gates_p.requires_grad:
                # cell (row, i) holds the gate of column sort_order[t, s] where pair_table[t, s] = row*quota + i
                by_col = torch.empty_like(ex["pair_table"]).scatter_(1, ex["sort_order"], ex["pair_table"])
                gate_rows = _SparseGateRowsEdge.apply(gates_p, by_col.reshape(-1), gate_rows)
        else:
            token_rows = []
            payload, mask, gate_rows, u_src, node_counts, inverse, u_node = general_hopa_planes(
                h.detach(), expert_idx, gates_p.detach(), world, n_experts, rpn, token_rows_out=token_rows)
            tok_table = token_rows[0]
            if gates_p.requires_grad:
                cells = inverse.view(T, k) * slots + expert_idx % slots
                gate_rows = _SparseGateRowsEdge.apply(gates_p, cells.reshape(-1), gate_rows)
        if h.requires_grad:
            payload = _FanOutEdge.apply(h, tok_table, payload)
        save_tensors.append(payload)      # seat 0
        save_tensors.append(gate_rows)    # seat 1

        # ---- Hop A (loop-back, outside the segments): what was packed for the wire is what arrives
        with torch.no_grad():
            if pack_mode == "small":
                sbuf, lay = _pk.hopa_pack_small(gate_rows.detach(), mask)
                if overlap_shared:
                    share_experts_output = shared_now()
                rgate, rmask = _pk.hopa_unpack_small(sbuf, lay)
                _pk.assert_not_aliased(sbuf, rgate, rmask)
                rx = payload.detach()
            elif pack_mode == "full":
                sbuf, lay = _pk.hopa_pack(payload.detach(), gate_rows.detach(), mask)
                if overlap_shared:
                    share_experts_output = shared_now()
                rx, rgate, rmask = _pk.hopa_unpack(sbuf, lay)
                _pk.assert_not_aliased(sbuf, rx, rgate, rmask)
            else:
                if overlap_shared:
                    share_experts_output = shared_now()
                rx, rmask, rgate = payload.detach(), mask, gate_rows.detach()

        # ---- segment 2: arrival chain, Hop B (loop-back) and expert order; graphs rooted at the two leaves
        rx_d = rx.detach().requires_grad_(True)
        rgate_d = rgate.detach().requires_grad_(True)
        R = rx_d.shape[0]
        with torch.no_grad():
            if quota is not None:
                exp_rx, gate_pairs, r_idx, slot_idx, _i_send, pair_pos = _ops.k1_arrival_raw(
                    rx_d, rmask, rgate_d, quota, epr, rpn, my_local, want_pair_pos=True)
            else:
                r_in, s_in = _expand_arrival(rmask, slots, None)
                _none, gate_pairs, r_idx, slot_idx, _i_send, _ordo = _ops.arrival_pairs(rx_d, r_in, s_in, rgate_d,
                                                                                        epr, rpn, move=False)
                per_row, _ = _ops.segment_table(r_idx, R, min(k, slots))
                exp_rx = _ops.scatter_rows(rx_d, per_row, r_idx.numel())      # each arrived row read once
            if pack_mode != "off":
                bbuf = _pk.hopb_pack_meta(slot_idx, gate_pairs)
                my_slot, my_gate = _pk.hopb_unpack_meta(bbuf, gate_pairs.dtype)
            else:
                my_slot, my_gate = slot_idx, gate_pairs
            permuted, order, tokens_per_expert, place, pprobs = _regroup_with_place(exp_rx, my_slot, slots, 0, my_gate)
            if quota is not None:
                red_table = _ops.index_chain(place, pair_pos).view(R, quota)
                cols = torch.arange(quota, device=h.device, dtype=torch.int64).unsqueeze(0).expand(R, quota).contiguous()
            else:
                red_table = _ops.index_chain(place, per_row)
                cols = _ops.index_chain(slot_idx, per_row)
        permuted = _FanOutEdge.apply(rx_d, red_table, permuted)
        pprobs = _GateCellsEdge.apply(rgate_d, red_table, cols, pprobs)
        save_tensors.append(None)         # seat 2
        save_tensors.append(rx_d)         # seat 3
        save_tensors.append(permuted)     # seat 4
        save_tensors.append(rgate_d)      # seat 5
        save_tensors.append(pprobs)       # seat 6
        if not overlap_shared:
            share_experts_output = shared_now()

    st = TA2AState()
    st.u_src, st.r_idx, st.order = u_src, r_idx, order
    st.R, st.T, st.hidden = R, T, H
    st.send_l = st.recv_l = st.is_l = st.ir_l = None
    st.intra, st.inter, st.dtype = intra_group, inter_group, hidden_states.dtype
    st.red_table, st.tok_table = red_table, tok_table
    st.where, st.token_of_place = _ops.pair_places(order, r_idx, my_slot, u_src, u_node, expert_idx, slots)
    return permuted, tokens_per_expert, pprobs, share_experts_output, st


def ta2a_unpermute_overlap(expert_out, st: TA2AState, save_tensors, out_shape=None):
    """Combine half of the overlap seam; returns ONE tensor.  Same math as :func:`ta2a_unpermute` (no gate
    multiply; a send row sums its pairs, a token sums its rows, fp32 accumulation and one rounding per level),
    cut at the return of Hop A: appends seats 7-9."""
    _hip.need_device(expert_out)
    with torch.enable_grad():
        eo_d = expert_out.detach().requires_grad_(True)
        with torch.no_grad():
            red = _ops.combine(eo_d, st.red_table, None, out_dtype=eo_d.dtype)
        red = _GatherReduceEdge.apply(eo_d, st.red_table, red)
        save_tensors.append(eo_d)         # seat 7
        save_tensors.append(red)          # seat 8
        back_d = red.detach().requires_grad_(True)          # Hop A back (loop-back), outside the segments
        with torch.no_grad():
            y = _ops.combine(back_d, st.tok_table, None, out_dtype=back_d.dtype)
        y = _GatherReduceEdge.apply(back_d, st.tok_table, y)
        if out_shape is not None:
            y = y.view(out_shape)
        save_tensors.append(back_d)       # seat 9
    return y

