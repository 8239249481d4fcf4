"""ctypes binding of libterrace_hip.so (the C ABI declared in include/terrace_hip.h).

torch is used for device memory and for the current HIP stream only; every computation on
the path is a kernel of the library.  There is no CPU or composed-torch fallback: a missing
library, or a tensor that is not on a ROCm device, raises.
"""
from __future__ import annotations

import ctypes
import glob
import os
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p

import torch

ENV_LIB = "TERRACE_OPS_LIB"
PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(os.path.dirname(PKG_DIR), "lib")

OK, EINVAL, ENOSPC, ELAUNCH, E2BIG = 0, -22, -28, -5, -7
F32, BF16, F16, FP8_B128 = 0, 1, 2, 3
MODE_CODES = {"full": 0, "group_limited": 1, "quota_only": 2, "global_topk": 3}
FORCE_GENERIC = 0x100
GATES_FLAG = {torch.float32: 0, torch.bfloat16: 0x200, torch.float16: 0x400}
PROBE_READ, PROBE_WRITE, PROBE_SUM8, PROBE_COPY = 0, 1, 2, 3
FAULT_ID_RANGE, FAULT_QUOTA, FAULT_FANOUT = 1, 2, 4
# enum terrace_dispatch_plane, in order
DISPATCH_PLANES = ("mask", "gate_rows", "u_src", "node_counts", "u_node", "inverse", "node_offsets", "pair_table",
                   "sort_order", "token_rows", "gate_sorted", "pair_src", "where", "status", "gate_pairs", "r_idx",
                   "slot_idx", "i_send", "pair_pos", "status_hopb", "order", "place", "kept", "tokens_per_expert",
                   "kept_per_expert", "status_regroup")
STATUS_WORDS = 4

_P, _I, _L, _Z = c_void_p, c_int, c_int64, c_size_t

# name -> (restype, argtypes); must list every function include/terrace_hip.h declares
SIGNATURES = {
    "terrace_version": (c_char_p, []),
    "terrace_strerror": (c_char_p, [_I]),
    "terrace_passthrough": (_I, [_P, _P, _Z, _P]),
    "terrace_stream_probe": (_I, [_I, _P, _P, _Z, _P]),
    "terrace_t_route": (_I, [_P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P]),
    "terrace_hist_workspace": (_Z, [_L, _I]),
    "terrace_hist": (_I, [_P, _L, _I, _P, _I, _P, _P, _Z, _P]),
    "terrace_argsort_small_workspace": (_Z, [_L, _I]),
    "terrace_argsort_small": (_I, [_P, _L, _I, _P, _P, _P, _P, _Z, _P]),
    "terrace_k2_pack_workspace": (_Z, [_L, _I, _I, _I]),
    "terrace_k2_pack": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _I, _I, _I,
                             _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_pack_quota_wire": (_I, [_P, _P, _P, _L, _I, _I, _L, _I, _I, _P, _P, _P, _P]),
    "terrace_k1_arrival_workspace": (_Z, [_L, _I, _I]),
    "terrace_k1_arrival": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _I, _I,
                                _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_regroup_workspace": (_Z, [_L, _I, _L]),
    "terrace_regroup": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _L,
                             _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P, _Z, _P]),
    "terrace_hopb_scatter_workspace": (_Z, [_L, _I, _I]),
    "terrace_hopb_scatter": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _I, _L,
                                  _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P, _Z, _P]),
    "terrace_hopb_scatter_move": (_I, [_P, _L, _L, _I, _I, _L, _P, _P, _Z, _P]),
    "terrace_gather_rows": (_I, [_P, _L, _P, _L, _L, _P, _P]),
    "terrace_scatter_rows": (_I, [_P, _P, _L, _I, _L, _P, _L, _P]),
    "terrace_index_chain": (_I, [_P, _L, _P, _L, _P, _P]),
    "terrace_index_chain2": (_I, [_P, _L, _P, _L, _P, _L, _P, _P]),
    "terrace_combine": (_I, [_P, _L, _I, _P, _P, _I, _L, _I, _L, _P, _I, _P]),
    "terrace_combine_pitched": (_I, [_P, _L, _I, _L, _P, _P, _I, _L, _I, _L, _P, _I, _P]),
    "terrace_combine_two_level": (_I, [_P, _L, _I, _P, _L, _I, _P, _L, _I, _L, _P, _I, _P]),
    "terrace_pack_planes": (_I, [_P, _L, _P, _L, _P, _L, _L, _L, _P, _P]),
    "terrace_unpack_planes": (_I, [_P, _L, _L, _P, _L, _P, _L, _P, _L, _P]),
    "terrace_k2_pack_wire": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _I, _I, _I,
                                  _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_k1_arrival_wire": (_I, [_P, _P, _I, _L, _L, _I, _I, _I, _I, _I,
                                     _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_regroup_wire": (_I, [_P, _P, _L, _L, _I, _I, _I, _L,
                                  _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_k2_pack_move": (_I, [_P, _L, _L, _I, _I, _I, _P, _P, _Z, _P]),
    "terrace_k1_arrival_move": (_I, [_P, _L, _L, _I, _I, _P, _P, _Z, _P]),
    "terrace_regroup_move": (_I, [_P, _L, _L, _I, _L, _P, _P, _Z, _P]),
    "terrace_plan_general_workspace": (_Z, [_L, _I, _I]),
    "terrace_plan_general": (_I, [_P, _L, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_build_mask": (_I, [_P, _P, _L, _I, _L, _P, _P, _P]),
    "terrace_scatter_elems": (_I, [_P, _I, _P, _P, _I, _L, _L, _I, _P, _P]),
    "terrace_expand_mask_quota": (_I, [_P, _L, _I, _I, _P, _P, _P]),
    "terrace_expand_mask_workspace": (_Z, [_L]),
    "terrace_expand_mask_count": (_I, [_P, _L, _I, _P, _P, _Z, _P]),
    "terrace_expand_mask_fill": (_I, [_P, _L, _I, _P, _P, _P, _P]),
    "terrace_arrival_pairs_workspace": (_Z, [_L, _I]),
    "terrace_arrival_pairs": (_I, [_P, _P, _P, _P, _L, _L, _L, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_segment_table_workspace": (_Z, [_L]),
    "terrace_segment_table": (_I, [_P, _L, _L, _I, _P, _P, _P, _Z, _P]),
    "terrace_pair_places": (_I, [_P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _L, _P, _P, _P, _P]),
    "terrace_routing_map_count": (_I, [_P, _L, _I, _P, _P]),
    "terrace_routing_map_topk": (_I, [_P, _P, _I, _L, _I, _I, _P, _P, _P]),
    "terrace_hopa_send_splits": (_I, [_P, _I, _I, _I, _P, _P]),
    "terrace_dispatch_workspace": (_Z, [_L, _I, _I, _I, _I, _I, _L, _I]),
    "terrace_dispatch": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _I, _I, _I, _L, _I, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "terrace_static_scratch_bytes": (_Z, []),
    "terrace_static_init": (_I, []),
    "terrace_k1_arrival_static": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _I, _I,
                                       _P, _P, _P, _P, _P, _P, _P, _P]),
}


class LibraryError(RuntimeError):
    """libterrace_hip.so could not be found or loaded, or lacks a declared symbol."""


_LIB = None
_LIB_PATH = None


def find_library() -> str:
    explicit = os.environ.get(ENV_LIB)
    if explicit:
        if not os.path.isfile(explicit):
            raise LibraryError(f"{ENV_LIB}={explicit} does not exist")
        return explicit
    hits = sorted(glob.glob(os.path.join(LIB_DIR, "libterrace_hip*.so")))
    if not hits:
        raise LibraryError(f"no libterrace_hip.so under {LIB_DIR}; build it with "
                           f"`python terracemoe-simulator_amd/csrc/build.py`")
    return hits[0]


def load(path: str | None = None):
    """Load (once) and type every entry point.  Raises LibraryError on any problem."""
    global _LIB, _LIB_PATH
    if _LIB is not None and (path is None or path == _LIB_PATH):
        return _LIB
    path = path or find_library()
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise LibraryError(f"dlopen({path}) failed: {e}") from e
    missing = [n for n in SIGNATURES if not hasattr(lib, n)]
    if missing:
        raise LibraryError(f"{path} lacks {missing}")
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _refuse_stale(lib, path)
    _LIB, _LIB_PATH = lib, path
    return lib


def _refuse_stale(lib, path):
    """In a source tree (csrc/build.py beside the package) the library must carry the digest of the sources
    that are there now: a kernel older than the host code that calls it can read what it was never given.
    ``TERRACE_ALLOW_STALE=1`` switches the check off; an installed package without sources has nothing to check."""
    build_py = os.path.join(os.path.dirname(PKG_DIR), "csrc", "build.py")
    if not os.path.exists(build_py) or os.environ.get("TERRACE_ALLOW_STALE") == "1":
        return
    import importlib.util
    spec = importlib.util.spec_from_file_location("terrace_csrc_build_check", build_py)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    stamped = lib.terrace_version().decode().rsplit("src:", 1)[-1]
    if stamped != mod.source_hash():
        raise LibraryError(f"{path} was built from other sources than those in {os.path.dirname(build_py)} "
                           f"(stamp {stamped}, sources {mod.source_hash()}): run python {build_py}")


def library_path():
    return _LIB_PATH


def unload_for_tests():
    global _LIB, _LIB_PATH
    _LIB = _LIB_PATH = None


def call(name: str, *args):
    rc = getattr(load(), name)(*args)
    if rc != OK:
        msg = load().terrace_strerror(rc).decode()
        raise RuntimeError(f"{name} failed: {msg} (status {rc})")


def query(name: str, *args) -> int:
    return int(getattr(load(), name)(*args))


def need_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("terrace (MI355X build): tensors must live on a ROCm device; this build has no "
                               "CPU path")


def ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream(device) -> c_void_p:
    """The HIP stream torch currently launches on for ``device``.  The raw-handle accessor is an order of
    magnitude cheaper than building a ``torch.cuda.Stream`` object, which matters where a step is a dozen
    launches of a few microseconds each."""
    if _RAW_STREAM is not None:
        index = device.index if isinstance(device, torch.device) else torch.device(device).index
        if index is None:
            index = torch.cuda.current_device()
        return c_void_p(_RAW_STREAM(index))
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def row_arg(t) -> int:
    """The ``row_bytes`` argument for a 2-D row tensor: its width in bytes, or -- for a row-pitched view (unit
    stride inside a row, rows further apart than they are wide) -- TERRACE_ROW_PITCHED(width, pitch)."""
    width = t.shape[1] * t.element_size()
    if t.shape[0] <= 1 or t.stride(0) == t.shape[1]:
        return width
    return width | ((t.stride(0) * t.element_size()) << 32)


def is_rows(t) -> bool:
    """Whether ``t`` can go to the library as it is: 2-D, unit stride inside a row, rows not overlapping."""
    return t.dim() == 2 and (t.shape[1] <= 1 or t.stride(1) == 1) and (t.shape[0] <= 1 or t.stride(0) >= t.shape[1])


def as_rows(t):
    """``t`` itself when it is packed or row-pitched, else a packed copy."""
    return t if t.is_contiguous() or is_rows(t) else t.contiguous()


def empty_rows(n: int, like):
    """[n, width] rows of ``like``'s dtype on ``like``'s device, on the same pitch as ``like``."""
    width = like.shape[1]
    if like.shape[0] <= 1 or like.stride(0) == width or not is_rows(like):
        return torch.empty((n, width), dtype=like.dtype, device=like.device)
    return torch.empty((n, like.stride(0)), dtype=like.dtype, device=like.device)[:, :width]


def float_code(dtype) -> int:
    try:
        return {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}[dtype]
    except KeyError:
        raise RuntimeError(f"unsupported floating dtype {dtype}") from None


def workspace(nbytes: int, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def new_status(device):
    return torch.empty(STATUS_WORDS, dtype=torch.int32, device=device)
