"""T-A2A wire containers on MI355X: several planes that share splits packed into one
int64-word row, and unpacked again.  Pure byte re-layout.

Same interface as the reference module (terrace/ta2a_pack.py there) for the packing itself:
``HopALayout`` / ``hopa_layout`` / ``hopa_pack`` / ``hopa_unpack``, ``HopASmallLayout`` /
``hopa_small_layout`` / ``hopa_pack_small`` / ``hopa_unpack_small``, ``hopb_meta_words`` /
``hopb_pack_meta`` / ``hopb_unpack_meta``, ``assert_not_aliased``, and the ``TERRACE_TA2A_PACK``
mode switch (``pack_mode`` / ``pack_enabled`` / ``reset``).  The exchange helpers of that module
(``hopa_exchange_*``, ``attach_edge``) wrap all-to-all collectives and are not part of a
one-GPU build.

Row layouts (int64 words, the id plane always leads so the float region starts on 8 bytes):
  Hop A full : [ids (id_w words) | payload (H) | gates (gw) | zero pad]   W = id_w + ceil((H+gw)/per_word)
  Hop A small: [ids (id_w words) | gates (gw) | zero pad]                 W = id_w + ceil(gw/per_word)
  Hop B meta : [slot id (1 word) | gate (1 element) | zero pad]           W = 2
Unpacked planes are freshly allocated dense tensors, never views of the container.
"""
from __future__ import annotations

import os

import torch

from . import _hip
from . import ops as _ops

_ENV_SWITCH = "TERRACE_TA2A_PACK"
_MODE: str | None = None
_MODE_OFF, _MODE_SMALL, _MODE_FULL = "off", "small", "full"
_ALIASES = {"0": _MODE_OFF, "off": _MODE_OFF, "no": _MODE_OFF,
            "1": _MODE_SMALL, "small": _MODE_SMALL, "meta": _MODE_SMALL,
            "full": _MODE_FULL, "2": _MODE_FULL, "all": _MODE_FULL}


def _env_mode() -> str:
    global _MODE
    if _MODE is None:
        raw = os.environ.get(_ENV_SWITCH)
        if raw is None:
            _MODE = _MODE_SMALL
        else:
            key = raw.strip().lower()
            if key not in _ALIASES:
                raise RuntimeError("%s=%r is not a valid mode. Valid values: %s. No silent fallback to the "
                                   "default." % (_ENV_SWITCH, raw, sorted(_ALIASES)))
            _MODE = _ALIASES[key]
    return _MODE


def pack_enabled() -> bool:
    return _env_mode() != _MODE_OFF


def pack_mode() -> str:
    """"off" / "small" / "full"; asks ``pack_enabled()`` first so a patched gate is honoured."""
    if not pack_enabled():
        return _MODE_OFF
    return _env_mode()


def reset() -> None:
    global _MODE
    _MODE = None


def _own(t: torch.Tensor) -> torch.Tensor:
    """Contiguous with storage of its own."""
    return t.clone(memory_format=torch.contiguous_format)


def _pack(planes, n: int, words: int, device):
    """planes: up to three (tensor, bytes per row); returns the [n, words] int64 container."""
    _ops._require()
    buf = torch.empty((n, words), dtype=torch.int64, device=device)
    args = []
    for t, nbytes in planes:
        args += [_hip.ptr(t), nbytes]
    while len(args) < 6:
        args += [None, 0]
    _hip.call("terrace_pack_planes", *args, n, words * 8, _hip.ptr(buf), _hip.stream(device))
    return buf


def _unpack(buf, outs):
    """outs: up to three (tensor or None, bytes per row), consecutive from the row head."""
    _ops._require()
    args = []
    for t, nbytes in outs:
        args += [_hip.ptr(t), nbytes]
    while len(args) < 6:
        args += [None, 0]
    _hip.call("terrace_unpack_planes", _hip.ptr(buf), buf.shape[1] * 8, buf.shape[0], *args, _hip.stream(buf.device))


# ---- Hop A, full container ---------------------------------------------------------------

class HopALayout:
    __slots__ = ("hidden", "gate_w", "id_w", "id_1d", "words", "dtype", "per_word")

    def __init__(self, hidden, gate_w, id_w, id_1d, dtype):
        self.hidden, self.gate_w = hidden, gate_w
        self.id_w, self.id_1d = id_w, id_1d
        self.dtype = dtype
        self.per_word = 8 // dtype.itemsize
        self.words = id_w + -(-(hidden + gate_w) // self.per_word)

    def __repr__(self):
        return (f"HopALayout(H={self.hidden}, gw={self.gate_w}, id_w={self.id_w}, "
                f"id_1d={self.id_1d}, words={self.words}, dtype={self.dtype})")


def hopa_layout(payload: torch.Tensor, gate_rows: torch.Tensor, ids: torch.Tensor) -> HopALayout:
    if payload.dtype != gate_rows.dtype:
        raise RuntimeError(f"Hop A packing requires payload/gate to share a dtype, got {payload.dtype} vs "
                           f"{gate_rows.dtype} -- the gate plane is derived from payload by contract")
    if ids.dtype != torch.int64:
        raise RuntimeError(f"Hop A packing's id plane must be int64, got {ids.dtype}")
    if ids.dim() not in (1, 2):
        raise RuntimeError(f"Hop A's id plane must be [n] or [n, quota], got {ids.shape}")
    id_1d = ids.dim() == 1
    id_w = 1 if id_1d else int(ids.shape[1])
    n = payload.shape[0]
    if ids.shape[0] != n or gate_rows.shape[0] != n:
        raise RuntimeError(f"Hop A's three planes must have equal row counts (they share splits), got "
                           f"payload={n} gate={gate_rows.shape[0]} id={ids.shape[0]}")
    return HopALayout(int(payload.shape[1]), int(gate_rows.shape[1]), id_w, id_1d, payload.dtype)


def hopa_pack(payload: torch.Tensor, gate_rows: torch.Tensor, ids: torch.Tensor):
    """([n, H] float, [n, gw] float, [n] / [n, quota] int64) -> ([n, W] int64, layout)."""
    lay = hopa_layout(payload, gate_rows, ids)
    _hip.need_device(payload, gate_rows, ids)
    payload, gate_rows, ids = payload.contiguous(), gate_rows.contiguous(), ids.contiguous()
    es = payload.element_size()
    buf = _pack([(ids, lay.id_w * 8), (payload, lay.hidden * es), (gate_rows, lay.gate_w * es)],
                payload.shape[0], lay.words, payload.device)
    return buf, lay


def hopa_unpack(buf: torch.Tensor, lay: HopALayout):
    """[n, W] int64 -> ([n, H] payload, [n, gw] gate, ids in their original shape), all dense."""
    _hip.need_device(buf)
    buf = buf.contiguous()
    n, dev, es = buf.shape[0], buf.device, lay.dtype.itemsize
    payload = torch.empty((n, lay.hidden), dtype=lay.dtype, device=dev)
    gate = torch.empty((n, lay.gate_w), dtype=lay.dtype, device=dev)
    ids = torch.empty((n,) if lay.id_1d else (n, lay.id_w), dtype=torch.int64, device=dev)
    _unpack(buf, [(ids, lay.id_w * 8), (payload, lay.hidden * es), (gate, lay.gate_w * es)])
    return payload, gate, ids


# ---- Hop A, small container (ids + gates; the payload travels alone) -------------------------

class HopASmallLayout:
    __slots__ = ("gate_w", "id_w", "id_1d", "words", "dtype", "per_word")

    def __init__(self, gate_w, id_w, id_1d, dtype):
        self.gate_w, self.id_w, self.id_1d = gate_w, id_w, id_1d
        self.dtype = dtype
        self.per_word = 8 // dtype.itemsize
        self.words = id_w + -(-gate_w // self.per_word)

    def __repr__(self):
        return (f"HopASmallLayout(gw={self.gate_w}, id_w={self.id_w}, id_1d={self.id_1d}, "
                f"words={self.words}, dtype={self.dtype})")


def hopa_small_layout(gate_rows: torch.Tensor, ids: torch.Tensor) -> HopASmallLayout:
    if ids.dtype != torch.int64:
        raise RuntimeError(f"Hop A small packing's id plane must be int64, got {ids.dtype}")
    if not gate_rows.is_floating_point():
        raise RuntimeError(f"Hop A small packing's gate plane must be floating point, got {gate_rows.dtype}")
    if ids.dim() not in (1, 2):
        raise RuntimeError(f"Hop A's id plane must be [n] or [n, quota], got {ids.shape}")
    if ids.shape[0] != gate_rows.shape[0]:
        raise RuntimeError(f"Hop A small packing's two planes must have equal row counts (they share splits), "
                           f"got gate={gate_rows.shape[0]} id={ids.shape[0]}")
    id_1d = ids.dim() == 1
    return HopASmallLayout(int(gate_rows.shape[1]), 1 if id_1d else int(ids.shape[1]), id_1d, gate_rows.dtype)


def hopa_pack_small(gate_rows: torch.Tensor, ids: torch.Tensor):
    """([n, gw] float, [n] / [n, quota] int64) -> ([n, Ws] int64, layout)."""
    lay = hopa_small_layout(gate_rows, ids)
    _hip.need_device(gate_rows, ids)
    gate_rows, ids = gate_rows.contiguous(), ids.contiguous()
    buf = _pack([(ids, lay.id_w * 8), (gate_rows, lay.gate_w * gate_rows.element_size())],
                gate_rows.shape[0], lay.words, gate_rows.device)
    return buf, lay


def hopa_unpack_small(buf: torch.Tensor, lay: HopASmallLayout):
    """[n, Ws] int64 -> ([n, gw] gate, ids in their original shape)."""
    _hip.need_device(buf)
    buf = buf.contiguous()
    n, dev = buf.shape[0], buf.device
    gate = torch.empty((n, lay.gate_w), dtype=lay.dtype, device=dev)
    ids = torch.empty((n,) if lay.id_1d else (n, lay.id_w), dtype=torch.int64, device=dev)
    _unpack(buf, [(ids, lay.id_w * 8), (gate, lay.gate_w * lay.dtype.itemsize)])
    return gate, ids


# ---- Hop B metadata container ---------------------------------------------------------------

def hopb_meta_words() -> int:
    return 2


def hopb_pack_meta(slot_idx: torch.Tensor, gate_pairs: torch.Tensor) -> torch.Tensor:
    """([P] int64 slot ids, [P] float gates) -> [P, 2] int64."""
    if slot_idx.dtype != torch.int64:
        raise RuntimeError(f"Hop B packing's id plane must be int64, got {slot_idx.dtype}")
    if slot_idx.shape != gate_pairs.shape:
        raise RuntimeError(f"Hop B packing requires both planes to share a shape (one scalar per pair), got "
                           f"{tuple(slot_idx.shape)} vs {tuple(gate_pairs.shape)}")
    if not gate_pairs.is_floating_point():
        raise RuntimeError(f"Hop B packing's gate plane must be floating point, got {gate_pairs.dtype}")
    _hip.need_device(slot_idx, gate_pairs)
    slot_idx, gate_pairs = slot_idx.contiguous(), gate_pairs.contiguous()
    return _pack([(slot_idx, 8), (gate_pairs, gate_pairs.element_size())], slot_idx.numel(), hopb_meta_words(),
                 slot_idx.device)


def hopb_unpack_meta(buf: torch.Tensor, dtype):
    """[P, 2] int64 -> ([P] int64 slot ids, [P] float gates)."""
    _hip.need_device(buf)
    buf = buf.contiguous()
    P, dev = buf.shape[0], buf.device
    slot = torch.empty((P,), dtype=torch.int64, device=dev)
    gate = torch.empty((P,), dtype=dtype, device=dev)
    _unpack(buf, [(slot, 8), (gate, dtype.itemsize)])
    return slot, gate


def assert_not_aliased(buf: torch.Tensor, *planes: torch.Tensor) -> None:
    """No unpacked plane may still point into ``buf`` when its storage is about to be released."""
    sp = buf.untyped_storage().data_ptr()
    for i, p in enumerate(planes):
        if p is not None and p.numel() and p.untyped_storage().data_ptr() == sp:
            raise RuntimeError(f"Unpacked plane {i} is still in shared storage with the pack buffer "
                               f"(shape={tuple(p.shape)}, buf={tuple(buf.shape)}) -- releasing the memory would "
                               f"leave it dangling.")
