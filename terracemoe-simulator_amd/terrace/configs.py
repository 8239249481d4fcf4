"""The five benchmark geometries of the dispatch/combine path and their synthetic inputs.

Inputs come from a CPU ``torch.Generator`` with a fixed seed per geometry, so a checker on
the host and the kernels on the device consume identical bits.  Nothing here computes any
stage of the path.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

FP8_BLOCK = 128
E4M3_MAX = 448.0


@dataclass(frozen=True)
class PathConfig:
    name: str
    T: int                 # tokens on this rank
    n_experts: int         # E
    n_groups: int          # N_g: routing groups == nodes
    top_k: int             # k
    top_groups: int        # M
    rpn: int               # cards per group
    hidden: int            # H
    fmt: str               # payload format: f32 | bf16 | fp8 (e4m3 rows with per-128 fp32 scales)
    bias: str = "none"     # none | normal (N(0, 0.1)) | zipf (s = 1.2 ranked, scaled to [0, 3])
    softmax_gates: bool = False     # gates = renormalised softmax over the selected experts
    capacity_factor: float | None = None
    seed: int = 1234
    row_pitch: int | None = None    # bytes between payload rows in every row buffer (None: rows back to back)

    @property
    def world(self) -> int:
        return self.n_groups * self.rpn

    @property
    def epr(self) -> int:
        return self.n_experts // self.world

    @property
    def slots(self) -> int:
        return self.epr * self.rpn

    @property
    def quota(self) -> int:
        return self.top_k // self.top_groups

    @property
    def send_rows(self) -> int:
        return self.T * self.top_groups

    @property
    def pairs(self) -> int:
        return self.T * self.top_k

    @property
    def row_bytes(self) -> int:
        if self.fmt == "f32":
            return self.hidden * 4
        if self.fmt == "bf16":
            return self.hidden * 2
        return self.hidden + 4 * (self.hidden // FP8_BLOCK)

    @property
    def gate_dtype(self):
        return torch.float32 if self.fmt == "f32" else torch.bfloat16

    @property
    def out_dtype(self):
        return torch.float32 if self.fmt == "f32" else torch.bfloat16

    def capacity(self, n_local: int) -> int | None:
        """Rows one local expert may keep: ceil(factor * pairs / n_local)."""
        if self.capacity_factor is None:
            return None
        return int(-(-self.capacity_factor * self.pairs // n_local))

    def scaled(self, T: int) -> "PathConfig":
        """Same geometry on fewer tokens (parity-test sizes)."""
        return PathConfig(**{**self.__dict__, "T": T})


CONFIGS = {
    "c1": PathConfig("c1_cpu_reference", 4096, 64, 8, 4, 2, 8, 1024, "f32", seed=1235),
    "c2": PathConfig("c2_deepseek_v3_slice", 16384, 256, 8, 8, 4, 8, 7168, "bf16", bias="normal",
                     softmax_gates=True, seed=1236),
    "c3": PathConfig("c3_high_dedup", 32768, 128, 16, 8, 2, 8, 4096, "bf16", seed=1237),
    "c4": PathConfig("c4_skewed_capacity", 65536, 256, 8, 8, 4, 8, 2048, "bf16", bias="zipf",
                     capacity_factor=1.25, seed=1238),
    # the 7392-byte fp8 row (codes, then the block scales) sits on an 8 KB pitch in every row buffer, so that the row
    # movers copy aligned kilobytes of it; the 800 bytes between one row's end and the next row are never touched
    "c5": PathConfig("c5_fp8_payload", 16384, 256, 8, 8, 4, 8, 7168, "fp8", bias="normal",
                     softmax_gates=True, seed=1239, row_pitch=8192),
}


def pitched_rows(rows: torch.Tensor, pitch_bytes: int | None) -> torch.Tensor:
    """The same [n, width] rows as a view of an [n, pitch] buffer (bytes past the width zero); unchanged when
    ``pitch_bytes`` is None."""
    if pitch_bytes is None:
        return rows
    n, width = rows.shape
    per = pitch_bytes // rows.element_size()
    assert per * rows.element_size() == pitch_bytes and per >= width
    base = torch.zeros((n, per), dtype=rows.dtype, device=rows.device)
    base[:, :width] = rows
    return base[:, :width]


def rows_to(rows: torch.Tensor, device) -> torch.Tensor:
    """``rows.to(device)`` that keeps a row pitch (a plain ``.to`` packs a view with gaps)."""
    if rows.dim() != 2 or rows.is_contiguous() or rows.shape[0] <= 1:
        return rows.to(device)
    n, width = rows.shape
    whole = rows.as_strided((n, rows.stride(0)), (rows.stride(0), 1))
    return whole.to(device)[:, :width]


def quantise_fp8_rows(x: torch.Tensor, pitch_bytes: int | None = None) -> torch.Tensor:
    """[n, H] float -> uint8 [n, H + H/32]: e4m3 codes then one fp32 scale per 128 elements
    (scale = max|x| / 448, or 1 for an all-zero block); on a row pitch when ``pitch_bytes`` is given."""
    n, hidden = x.shape
    xb = x.float().reshape(n, hidden // FP8_BLOCK, FP8_BLOCK)
    amax = xb.abs().amax(-1)
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax))
    codes = (xb / scale[..., None]).to(torch.float8_e4m3fn).view(torch.uint8).reshape(n, hidden)
    return pitched_rows(torch.cat([codes, scale.contiguous().view(torch.uint8).reshape(n, -1)], dim=1).contiguous(),
                        pitch_bytes)


def make_inputs(cfg: PathConfig) -> dict:
    """CPU tensors: logits [T,E] f32, bias [E] f32, gate_affinity [T,E] f32 or None,
    x (payload rows in storage form: f32 / bf16 [T,H] or uint8 [T,row_bytes]; a view of a wider buffer when the
    geometry names a row pitch -- move it with ``rows_to``)."""
    g = torch.Generator().manual_seed(cfg.seed)
    logits = torch.randn(cfg.T, cfg.n_experts, generator=g)
    if cfg.bias == "normal":
        bias = torch.randn(cfg.n_experts, generator=g) * 0.1
    elif cfg.bias == "zipf":
        ranks = torch.randperm(cfg.n_experts, generator=g).float() + 1.0
        w = ranks.pow(-1.2)
        bias = 3.0 * (w - w.min()) / (w.max() - w.min())
    else:
        bias = torch.zeros(cfg.n_experts)
    gate_aff = None
    if cfg.softmax_gates:
        gate_aff = torch.exp(logits - logits.max(-1, keepdim=True).values)
    x32 = torch.randn(cfg.T, cfg.hidden, generator=g)
    if cfg.fmt == "f32":
        x = x32
    elif cfg.fmt == "bf16":
        x = x32.to(torch.bfloat16)
    else:
        x = quantise_fp8_rows(x32)
    return {"logits": logits, "bias": bias, "gate_affinity": gate_aff, "x": pitched_rows(x, cfg.row_pitch)}


def algorithmic_bytes(cfg: PathConfig, out_row_bytes: int | None = None) -> dict:
    """Bytes each stage has to move, counting every payload row once on the read side and once
    on the write side of the stage (the reference's convention for its row-gather bandwidth),
    plus the index and gate planes."""
    T, E, k, M, q = cfg.T, cfg.n_experts, cfg.top_k, cfg.top_groups, cfg.quota
    S, P, row = cfg.send_rows, cfg.pairs, cfg.row_bytes
    gb = 4 if cfg.fmt == "f32" else 2
    orow = out_row_bytes if out_row_bytes is not None else cfg.hidden * (4 if cfg.fmt == "f32" else 2)
    crow = row                       # combine reads rows in the payload format
    return {
        "route": T * E * 4 + E * 4 + T * (k * 8 + k * 4 + M * 8),
        "pack": 2 * S * row + T * k * 8 + (S + T * k + cfg.n_groups) * 8 + S * q * (8 + gb) + T * k * (8 + gb),
        "arrival": 2 * P * row + P * (8 + 8 + gb) + S * q * (8 + gb),
        "regroup": 2 * P * row + P * 8 * 2,
        "combine": P * crow + P * 4 + P * 8 + T * orow,
    }


def minimum_traffic_bytes(cfg: PathConfig, kept_pairs: int | None = None, places: int | None = None) -> dict:
    """HBM bytes each stage cannot avoid: every distinct payload row read once and every output row
    written once (a scatter reads a source row once however many copies it writes), plus the same
    index and gate planes as ``algorithmic_bytes``.  ``kept_pairs`` / ``places`` describe a capacity
    layout (rows that survive the cut, rows of the padded buffer); default: drop-less."""
    T, S, P, row = cfg.T, cfg.send_rows, cfg.pairs, cfg.row_bytes
    kept = P if kept_pairs is None else kept_pairs
    places = P if places is None else places
    alg = algorithmic_bytes(cfg)
    return {
        "route": alg["route"],
        "pack": alg["pack"] - 2 * S * row + (T + S) * row,
        "arrival": alg["arrival"] - 2 * P * row + (S + P) * row,
        "regroup": alg["regroup"] - 2 * P * row + (kept + places) * row,
        "combine": alg["combine"] - P * row + kept * row,
    }


def onepass_traffic_bytes(cfg: PathConfig, places: int | None = None) -> int:
    """HBM bytes the one-pass Hop-B scatter cannot avoid: every arrived row read once, every row of the
    expert-order buffer written once (kept rows and zero padding rows alike), the slot table read and the
    place / tag planes written."""
    S, P, row = cfg.send_rows, cfg.pairs, cfg.row_bytes
    places = P if places is None else places
    return (S + places) * row + P * 8 + P * (8 + 8 + 8)

