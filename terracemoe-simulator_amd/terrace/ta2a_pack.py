"""T-A2A wire containers on MI355X: planes that travel with the same splits, laid side by side in rows of
int64 words by one kernel, and split again by another.  Pure byte re-layout.

The module keeps the reference module's names (terrace/ta2a_pack.py there): ``HopALayout`` / ``hopa_layout`` /
``hopa_pack`` / ``hopa_unpack``, ``HopASmallLayout`` / ``hopa_small_layout`` / ``hopa_pack_small`` /
``hopa_unpack_small``, ``hopb_meta_words`` / ``hopb_pack_meta`` / ``hopb_unpack_meta``, ``assert_not_aliased``
and the ``TERRACE_TA2A_PACK`` switch (``pack_mode`` / ``pack_enabled`` / ``reset``).  Its exchange helpers
(``hopa_exchange_*``, ``attach_edge``) wrap all-to-all collectives and have no place in a one-GPU build.

A container row is a run of regions, ids first so that the floating-point region starts on an 8-byte boundary,
zero padded to whole words:

  Hop A full   ids (id_w words) | payload (H elements) | gates (gw elements)     W = id_w + ceil((H + gw) / per_word)
  Hop A small  ids (id_w words) | gates (gw elements)                            W = id_w + ceil(gw / per_word)
  Hop B meta   slot id (1 word) | gate (1 element)                               W = 2

with ``per_word = 8 // itemsize``.  Every unpacked plane is a dense tensor with storage of its own: the kernel
writes it, nothing is ever a view of the container.
"""
from __future__ import annotations

import os

import torch

from . import _hip
from . import ops as _ops

_ENV_SWITCH = "TERRACE_TA2A_PACK"

# spelling accepted in the environment -> mode
_SPELLINGS = {**dict.fromkeys(("0", "off", "no"), "off"),
              **dict.fromkeys(("1", "small", "meta"), "small"),
              **dict.fromkeys(("2", "full", "all"), "full")}
_cached_mode: list = []          # empty: environment not read yet; else [mode]


def _mode_from_environment() -> str:
    """The switch is read once; an unknown spelling raises rather than meaning the default."""
    if not _cached_mode:
        raw = os.environ.get(_ENV_SWITCH)
        mode = "small" if raw is None else _SPELLINGS.get(raw.strip().lower())
        if mode is None:
            raise RuntimeError(f"{_ENV_SWITCH}={raw!r} is not a valid mode (valid: {sorted(_SPELLINGS)}); "
                               f"refusing to fall back to the default silently")
        _cached_mode.append(mode)
    return _cached_mode[0]


def pack_enabled() -> bool:
    return _mode_from_environment() != "off"


def pack_mode() -> str:
    """"off", "small" or "full".  Goes through ``pack_enabled()`` so that a caller who patches that gate is obeyed."""
    return _mode_from_environment() if pack_enabled() else "off"


def reset() -> None:
    """Forget the cached switch (test hook)."""
    _cached_mode.clear()


# ---- the two kernels --------------------------------------------------------------------------

def _three(regions):
    """[(tensor or None, bytes per row), ...] -> the six pointer / width arguments of the plane kernels."""
    flat = []
    for tensor, width in regions:
        flat += [_hip.ptr(tensor), width]
    return flat + [None, 0] * (3 - len(regions))


def _lay_side_by_side(regions, n_rows: int, words: int, device) -> torch.Tensor:
    _ops._require()
    out = torch.empty((n_rows, words), dtype=torch.int64, device=device)
    _hip.call("terrace_pack_planes", *_three(regions), n_rows, words * 8, _hip.ptr(out), _hip.stream(device))
    return out


def _split(container: torch.Tensor, regions) -> None:
    _ops._require()
    _hip.call("terrace_unpack_planes", _hip.ptr(container), container.shape[1] * 8, container.shape[0],
              *_three(regions), _hip.stream(container.device))


# ---- layouts ------------------------------------------------------------------------------------

def _id_plane_shape(ids: torch.Tensor, what: str):
    """(id_w, id_1d) of an id plane: [n] (one mask word per row) or [n, quota] (a slot table)."""
    if ids.dtype != torch.int64:
        raise RuntimeError(f"{what}: the id plane must be int64, got {ids.dtype}")
    if ids.dim() == 1:
        return 1, True
    if ids.dim() == 2:
        return int(ids.shape[1]), False
    raise RuntimeError(f"{what}: the id plane must have shape [n] or [n, quota], got {tuple(ids.shape)}")


def _same_rows(what: str, **planes):
    counts = {name: int(t.shape[0]) for name, t in planes.items()}
    if len(set(counts.values())) > 1:
        raise RuntimeError(f"{what}: planes that share splits must have one row count, got {counts}")


class HopALayout:
    """Geometry of a full Hop-A container row; ``words`` is its width in int64 words."""
    __slots__ = ("hidden", "gate_w", "id_w", "id_1d", "words", "dtype", "per_word")

    def __init__(self, hidden, gate_w, id_w, id_1d, dtype):
        self.hidden, self.gate_w, self.id_w, self.id_1d, self.dtype = hidden, gate_w, id_w, id_1d, dtype
        self.per_word = 8 // dtype.itemsize
        self.words = id_w + (hidden + gate_w + self.per_word - 1) // self.per_word

    def __repr__(self):
        fields = ", ".join(f"{name}={getattr(self, name)}" for name in ("hidden", "gate_w", "id_w", "id_1d", "words",
                                                                        "dtype"))
        return f"HopALayout({fields})"


class HopASmallLayout:
    """Geometry of a small Hop-A container row (ids and gates; the payload travels on its own)."""
    __slots__ = ("gate_w", "id_w", "id_1d", "words", "dtype", "per_word")

    def __init__(self, gate_w, id_w, id_1d, dtype):
        self.gate_w, self.id_w, self.id_1d, self.dtype = gate_w, id_w, id_1d, dtype
        self.per_word = 8 // dtype.itemsize
        self.words = id_w + (gate_w + self.per_word - 1) // self.per_word

    def __repr__(self):
        fields = ", ".join(f"{name}={getattr(self, name)}" for name in ("gate_w", "id_w", "id_1d", "words", "dtype"))
        return f"HopASmallLayout({fields})"


def hopa_layout(payload: torch.Tensor, gate_rows: torch.Tensor, ids: torch.Tensor) -> HopALayout:
    what = "Hop A container"
    if gate_rows.dtype != payload.dtype:
        raise RuntimeError(f"{what}: the gate plane is derived from the payload and must share its dtype, got "
                           f"{gate_rows.dtype} beside {payload.dtype}")
    id_w, id_1d = _id_plane_shape(ids, what)
    _same_rows(what, payload=payload, gate=gate_rows, id=ids)
    return HopALayout(int(payload.shape[1]), int(gate_rows.shape[1]), id_w, id_1d, payload.dtype)


def hopa_small_layout(gate_rows: torch.Tensor, ids: torch.Tensor) -> HopASmallLayout:
    what = "Hop A small container"
    id_w, id_1d = _id_plane_shape(ids, what)
    if not gate_rows.is_floating_point():
        raise RuntimeError(f"{what}: the gate plane must be floating point, got {gate_rows.dtype}")
    _same_rows(what, gate=gate_rows, id=ids)
    return HopASmallLayout(int(gate_rows.shape[1]), id_w, id_1d, gate_rows.dtype)


def _new_ids(lay, n_rows: int, device) -> torch.Tensor:
    return torch.empty((n_rows,) if lay.id_1d else (n_rows, lay.id_w), dtype=torch.int64, device=device)


# ---- Hop A -----------------------------------------------------------------------------------------

def hopa_pack(payload: torch.Tensor, gate_rows: torch.Tensor, ids: torch.Tensor):
    """([n, H] float, [n, gw] float, [n] / [n, quota] int64) -> ([n, W] int64 container, its layout)."""
    lay = hopa_layout(payload, gate_rows, ids)
    _hip.need_device(payload, gate_rows, ids)
    size = payload.element_size()
    regions = [(ids.contiguous(), 8 * lay.id_w), (payload.contiguous(), size * lay.hidden),
               (gate_rows.contiguous(), size * lay.gate_w)]
    return _lay_side_by_side(regions, payload.shape[0], lay.words, payload.device), lay


def hopa_unpack(buf: torch.Tensor, lay: HopALayout):
    """[n, W] int64 -> ([n, H] payload, [n, gw] gates, ids in the shape they were packed from)."""
    _hip.need_device(buf)
    buf = buf.contiguous()
    n, dev, size = buf.shape[0], buf.device, lay.dtype.itemsize
    ids = _new_ids(lay, n, dev)
    payload = torch.empty((n, lay.hidden), dtype=lay.dtype, device=dev)
    gates = torch.empty((n, lay.gate_w), dtype=lay.dtype, device=dev)
    _split(buf, [(ids, 8 * lay.id_w), (payload, size * lay.hidden), (gates, size * lay.gate_w)])
    return payload, gates, ids


def hopa_pack_small(gate_rows: torch.Tensor, ids: torch.Tensor):
    """([n, gw] float, [n] / [n, quota] int64) -> ([n, Ws] int64 container, its layout)."""
    lay = hopa_small_layout(gate_rows, ids)
    _hip.need_device(gate_rows, ids)
    regions = [(ids.contiguous(), 8 * lay.id_w), (gate_rows.contiguous(), gate_rows.element_size() * lay.gate_w)]
    return _lay_side_by_side(regions, gate_rows.shape[0], lay.words, gate_rows.device), lay


def hopa_unpack_small(buf: torch.Tensor, lay: HopASmallLayout):
    """[n, Ws] int64 -> ([n, gw] gates, ids in the shape they were packed from)."""
    _hip.need_device(buf)
    buf = buf.contiguous()
    n, dev = buf.shape[0], buf.device
    ids = _new_ids(lay, n, dev)
    gates = torch.empty((n, lay.gate_w), dtype=lay.dtype, device=dev)
    _split(buf, [(ids, 8 * lay.id_w), (gates, lay.dtype.itemsize * lay.gate_w)])
    return gates, ids


# ---- Hop B -----------------------------------------------------------------------------------------

def hopb_meta_words() -> int:
    """One word for the slot id, one that starts with the gate."""
    return 2


def hopb_pack_meta(slot_idx: torch.Tensor, gate_pairs: torch.Tensor) -> torch.Tensor:
    """([P] int64 slot ids, [P] float gates) -> [P, 2] int64."""
    what = "Hop B container"
    if slot_idx.dtype != torch.int64:
        raise RuntimeError(f"{what}: the id plane must be int64, got {slot_idx.dtype}")
    if not gate_pairs.is_floating_point():
        raise RuntimeError(f"{what}: the gate plane must be floating point, got {gate_pairs.dtype}")
    if tuple(slot_idx.shape) != tuple(gate_pairs.shape):
        raise RuntimeError(f"{what}: one slot id and one gate per pair, so both planes must have one shape; got "
                           f"{tuple(slot_idx.shape)} and {tuple(gate_pairs.shape)}")
    _hip.need_device(slot_idx, gate_pairs)
    regions = [(slot_idx.contiguous(), 8), (gate_pairs.contiguous(), gate_pairs.element_size())]
    return _lay_side_by_side(regions, slot_idx.numel(), hopb_meta_words(), slot_idx.device)


def hopb_unpack_meta(buf: torch.Tensor, dtype):
    """[P, 2] int64 -> ([P] int64 slot ids, [P] gates of ``dtype``)."""
    _hip.need_device(buf)
    buf = buf.contiguous()
    slots = torch.empty((buf.shape[0],), dtype=torch.int64, device=buf.device)
    gates = torch.empty((buf.shape[0],), dtype=dtype, device=buf.device)
    _split(buf, [(slots, 8), (gates, dtype.itemsize)])
    return slots, gates


def assert_not_aliased(buf: torch.Tensor, *planes: torch.Tensor) -> None:
    """Tripwire for a caller about to release ``buf``'s memory: none of the planes unpacked from it may still live
    in its storage."""
    home = buf.untyped_storage().data_ptr()
    for position, plane in enumerate(planes):
        if plane is None or plane.numel() == 0:
            continue
        if plane.untyped_storage().data_ptr() == home:
            raise RuntimeError(f"unpacked plane {position} (shape {tuple(plane.shape)}) still shares storage with the "
                               f"container (shape {tuple(buf.shape)}): releasing the container would leave it dangling")
