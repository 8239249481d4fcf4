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
        red = _ops.combine(expert_out, red_table, None, out_dtype=expert_out.dtype)
        return _ops.combine(red, tok_table, None, out_dtype=out_dtype)

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
        payload, mask, gate_rows, u_src, node_counts, _inverse, u_node = general_hopa_planes(
            hidden_states, expert_idx, gates, world, n_experts, rpn)

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
        node_rx, my_meta, r_idx, _i_send, pair_pos = _ops.k1_arrival_wire(rx, rwire, gates.dtype, quota, epr, rpn,
                                                                          my_local)
        my_slot = my_meta[:, 0]
        permuted, order, tokens_per_expert, place, pprobs = _ops.regroup_wire(node_rx, my_meta, gates.dtype, slots, 0)
    else:
        if quota is not None:
            exp_rx, gate_pairs, r_idx, slot_idx, _i_send, pair_pos = _ops.k1_arrival_raw(
                rx, rmask, rgate, quota, epr, rpn, my_local, want_pair_pos=True)
        else:
            r_in, s_in = _expand_arrival(rmask, slots, None)
            exp_rx, gate_pairs, r_idx, slot_idx, _i_send, _ordo = _ops.arrival_pairs(rx, r_in, s_in, rgate, epr, rpn)
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
        per_row, _ = _ops.segment_table(r_idx, R, min(k, slots))
        st.red_table = _ops.index_chain(place, per_row)
        st.tok_table, _ = _ops.segment_table(u_src, T, min(k, n_nodes))
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
    red = _ops.combine(expert_out, st.red_table, None, out_dtype=expert_out.dtype)
    return _ops.combine(red, st.tok_table, None, out_dtype=out_like.dtype)
