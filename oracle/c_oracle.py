"""ctypes face of oracle/terrace_oracle.c (numpy arrays in, numpy arrays out).

TEST INFRASTRUCTURE: used by tests/test_oracle_c.py (pinned bit for bit to the numpy oracle)
and by bench.py's cpu_baseline leg.  Row payloads and gate planes are passed as raw bytes.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_c", "libterrace_oracle.so")
_LIB = None
FMT = {"f32": 0, "bf16": 1, "fp8": 3}


def available() -> bool:
    return os.path.isfile(LIB_PATH)


def lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(LIB_PATH)
        _LIB.orc_k2_pack.restype = ctypes.c_int
        _LIB.orc_threads.restype = ctypes.c_int
    return _LIB


def _p(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


def _i64(x):
    return ctypes.c_int64(int(x))


def threads() -> int:
    return int(lib().orc_threads())


def t_route(aff, bias, E, Ng, k, M, pool=2, gate_affinity=None):
    aff = np.ascontiguousarray(aff, np.float32)
    bias = np.ascontiguousarray(bias, np.float32)
    ga = None if gate_affinity is None else np.ascontiguousarray(gate_affinity, np.float32)
    T = aff.shape[0]
    e = np.empty((T, k), np.int64)
    g = np.empty((T, k), np.float32)
    grp = np.empty((T, M), np.int64)
    lib().orc_route_full(_p(aff), _p(bias), _p(ga), _i64(T), E, Ng, k, M, pool, _p(e), _p(g), _p(grp))
    return e, g, grp


def k2_pack(hidden, expert_idx, gates, world, n_experts, rpn, M):
    """Returns (payload, mask, gate_rows, u_src, counts, extras) or raises ValueError."""
    hidden = np.ascontiguousarray(hidden)
    gates = np.ascontiguousarray(gates)
    e = np.ascontiguousarray(expert_idx, np.int64)
    T, k = e.shape
    S, q, n_nodes = T * M, k // M, world // rpn
    payload = np.empty((S,) + hidden.shape[1:], hidden.dtype)
    mask = np.empty((S, q), np.int64)
    gate_rows = np.empty((S, q), gates.dtype)
    u_src, u_node, counts = np.empty(S, np.int64), np.empty(S, np.int64), np.empty(n_nodes, np.int64)
    inverse, pair_table, sort_order = np.empty(T * k, np.int64), np.empty((T, k), np.int64), np.empty((T, k), np.int64)
    rc = lib().orc_k2_pack(_p(hidden), _p(e), _p(gates), _i64(T), _i64(hidden.strides[0]), gates.itemsize, k, world,
                           n_experts, rpn, M, _p(payload), _p(mask), _p(gate_rows), _p(u_src), _p(counts), _p(u_node),
                           _p(inverse), _p(pair_table), _p(sort_order))
    if rc:
        raise ValueError("k2_pack: routing is not equal-quota over exactly M nodes (or an id is out of range)")
    return payload, mask, gate_rows, u_src, counts, {"u_node": u_node, "inverse": inverse, "pair_table": pair_table,
                                                     "sort_order": sort_order}


def k1_arrival(rx, rslot, rgate, quota, epr, rpn):
    rx, rgate = np.ascontiguousarray(rx), np.ascontiguousarray(rgate)
    rslot = np.ascontiguousarray(rslot, np.int64)
    R = rslot.shape[0]
    P = R * quota
    send = np.empty((P,) + rx.shape[1:], rx.dtype)
    gp = np.empty(P, rgate.dtype)
    r_idx, s_idx, pos = np.empty(P, np.int64), np.empty(P, np.int64), np.empty(P, np.int64)
    i_send = np.empty(rpn, np.int64)
    row_bytes = rx.strides[0] if R else 0
    lib().orc_k1_arrival(_p(rx), _p(rslot), _p(rgate), _i64(R), _i64(row_bytes), rgate.itemsize, quota, epr, rpn,
                         _p(send), _p(gp), _p(r_idx), _p(s_idx), _p(i_send), _p(pos))
    return send, gp, r_idx, s_idx, i_send, pos


def regroup(node_rx, my_slot, epr, my_local=0, capacity=None):
    node_rx = np.ascontiguousarray(node_rx)
    my_slot = np.ascontiguousarray(my_slot, np.int64).reshape(-1)
    P = my_slot.size
    cap = -1 if capacity is None else int(capacity)
    places = P if capacity is None else epr * cap
    permuted = np.empty((places,) + node_rx.shape[1:], node_rx.dtype)
    place, kept, tpe = np.empty(P, np.int64), np.empty(P, np.uint8), np.empty(epr, np.int64)
    row_bytes = node_rx.strides[0] if P else 0
    lib().orc_regroup(_p(node_rx), _p(my_slot), _i64(P), _i64(row_bytes), epr, my_local, _i64(cap), _p(permuted),
                      _p(place), _p(kept), _p(tpe))
    return permuted, place, kept.astype(bool), tpe


def combine(src_rows, idx, weights, in_fmt="f32", out_fmt="f32", hidden=None):
    src_rows = np.ascontiguousarray(src_rows)
    idx = np.ascontiguousarray(idx, np.int64)
    w = None if weights is None else np.ascontiguousarray(weights, np.float32)
    n_out, fan = idx.shape
    hidden = int(hidden if hidden is not None else src_rows.shape[1])
    out = np.empty((n_out, hidden), np.float32 if out_fmt == "f32" else np.uint16)
    lib().orc_combine(_p(src_rows), FMT[in_fmt], _p(idx), _p(w), _i64(n_out), fan, _i64(hidden), _p(out), FMT[out_fmt])
    return out
