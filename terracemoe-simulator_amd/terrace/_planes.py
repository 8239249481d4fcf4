"""Many small device planes out of one allocation.

A dispatch writes some thirty index and gate planes.  Allocating each with ``torch.empty`` costs the host more than
the kernels that fill them cost the GPU on a small batch, so the loop-back dispatch takes ONE byte slab from torch's
allocator, hands the library raw addresses inside it, and only builds a tensor view of a plane when somebody
reads it.  The arrangement of the planes depends on the geometry alone and is computed once per geometry; a step
then creates a handful of Python objects, not dozens (every container object a step creates brings the interpreter's
cyclic collector closer to a full pass, which stalls the host for tens of milliseconds).  Nothing here touches device
memory.
"""
from __future__ import annotations

from ctypes import c_void_p

import torch

_ALIGN = 256
_ITEM = {torch.int64: 8, torch.int32: 4, torch.float32: 4, torch.bfloat16: 2, torch.float16: 2, torch.uint8: 1,
         torch.bool: 1}
_LAZY = object()          # placeholder of a plane nobody has read yet


class Layout:
    """Where each named plane sits in the slab: name -> (offset, shape, dtype, nbytes)."""
    __slots__ = ("at", "total", "offsets")

    def __init__(self, planes):
        """planes: iterable of (name, shape, dtype); a None shape leaves the name out."""
        self.at, self.total, self.offsets = {}, 0, None
        for name, shape, dtype in planes:
            if shape is None:
                continue
            n = _ITEM[dtype]
            for d in shape:
                n *= int(d)
            self.at[name] = (self.total, tuple(int(d) for d in shape), dtype, n)
            self.total += (max(n, 1) + _ALIGN - 1) // _ALIGN * _ALIGN


class Slab:
    """One ``torch.empty`` of bytes arranged by a Layout."""
    __slots__ = ("buf", "base", "layout")

    def __init__(self, layout: Layout, device):
        self.layout = layout
        self.buf = torch.empty(max(layout.total, _ALIGN), dtype=torch.uint8, device=device)
        self.base = self.buf.data_ptr()

    def ptr(self, name):
        """Device address of a plane for the library, or None for a plane the layout leaves out."""
        entry = self.layout.at.get(name)
        return None if entry is None else c_void_p(self.base + entry[0])

    def nbytes(self, name) -> int:
        return self.layout.at[name][3]

    def tensor(self, name) -> torch.Tensor:
        offset, shape, dtype, n = self.layout.at[name]
        flat = self.buf[offset:offset + n]
        if dtype == torch.bool:
            return flat.view(shape).view(torch.bool)
        return flat.view(dtype).view(shape)


class LazyDict(dict):
    """The planes of a slab whose names start with ``prefix``, as a dict that builds a tensor when a key is first
    read (keys without a plane hold ordinary values)."""

    def __init__(self, slab: Slab, prefix: str):
        dict.__init__(self, {name[len(prefix):]: _LAZY for name in slab.layout.at if name.startswith(prefix)})
        self._slab, self._prefix = slab, prefix

    def __getitem__(self, key):
        value = dict.__getitem__(self, key)
        if value is _LAZY:
            value = self._slab.tensor(self._prefix + key)
            dict.__setitem__(self, key, value)
        return value

    def get(self, key, default=None):
        return self[key] if key in self else default

    def values(self):
        return [self[k] for k in self]

    def items(self):
        return [(k, self[k]) for k in self]


class LazyFields:
    """Attribute bag over explicit values and the planes of a slab (a plane turns into a tensor when first read;
    a plane the layout leaves out reads as None)."""

    def __init__(self, slab: Slab | None = None, optional=(), **fields):
        object.__setattr__(self, "_fields", fields)
        object.__setattr__(self, "_slab", slab)
        object.__setattr__(self, "_optional", optional)

    def __getattr__(self, name):
        fields = object.__getattribute__(self, "_fields")
        if name in fields:
            return fields[name]
        slab = object.__getattribute__(self, "_slab")
        if slab is not None and name in slab.layout.at:
            value = fields[name] = slab.tensor(name)
            return value
        if name in object.__getattribute__(self, "_optional"):
            return None
        raise AttributeError(name)

    def __setattr__(self, name, value):
        object.__getattribute__(self, "_fields")[name] = value
