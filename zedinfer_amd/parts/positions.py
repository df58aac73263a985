"""Position encodings.  They act where queries and keys leave the projection; the mixer stores what they made."""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch

from .. import ops
from ..config.forward_config import PartSpec
from .base import PositionEncoding, Runtime, register_position_encoding


def stretched_frequencies(rotary_dim: int, theta: float, scaling) -> np.ndarray:
    """f_i = theta^(-2i / rotary_dim) in double precision, with the frequencies of long wavelengths divided:
    with wavelength l = 2 pi / f, f stays where l < original / high, becomes f / factor where l > original / low,
    and between the two is (1 - s) f / factor + s f with s = (original / l - low) / (high - low).  Rounded to
    float32 once, at the end."""
    missing = [k for k in ("factor", "low", "high", "original") if k not in scaling]
    if missing:
        raise ValueError("rope scaling lacks " + ", ".join(missing))
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    if not (factor > 0 and high > low and orig > 0):
        raise ValueError("rope scaling: factor and original must be positive, high above low")
    i = np.arange(rotary_dim // 2, dtype=np.float64)
    f = np.power(float(theta), -2.0 * i / rotary_dim)
    wavelength = 2.0 * np.pi / f
    s = (orig / wavelength - low) / (high - low)
    mixed = (1.0 - s) * f / factor + s * f
    out = np.where(wavelength < orig / high, f, np.where(wavelength > orig / low, f / factor, mixed))
    return out.astype(np.float32)


@register_position_encoding("rope_neox")
class RopeNeox(PositionEncoding):
    """Split-half rotary encoding: pairs (k, k + R/2) of the first R = ``rotary_dim`` dims of
    each head turn by pos * theta^(-2k/R) (reference: src/backend/ops/rope/cpu/rope_cpu.cpp:12-66;
    the reference rotates the whole head, no scaling: rope_nvidia.cu:50).
    params: head_dim, theta, rotary_dim (default head_dim), scaling (None, or a dict factor / low / high /
    original: long wavelengths are stretched, ``stretched_frequencies``)."""

    graph_safe = True
    tape_safe = True

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.head_dim = int(spec.params["head_dim"])
        self.rotary_dim = int(spec.params.get("rotary_dim", self.head_dim))
        self.theta = float(spec.params["theta"])
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rope_neox: rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        scaling = spec.params.get("scaling")
        self.scaling = tuple(sorted((str(k), float(v)) for k, v in scaling.items())) if scaling else None
        if self.scaling is None:
            self.inv_freq = ops.rope_inv_freq(self.rotary_dim, self.theta, rt.device)
        else:
            self.inv_freq = torch.from_numpy(stretched_frequencies(self.rotary_dim, self.theta, dict(self.scaling))).to(rt.device)

    def step_table(self, batch):
        key = ("rope_neox", self.rotary_dim, self.theta, self.scaling)
        table = batch.shared.get(key)
        if table is None:
            out = self.rt.buffer(f"rope_table_{self.rotary_dim}_{self.theta!r}_{self.scaling!r}",
                                 (batch.num_tokens, self.rotary_dim // 2, 2), torch.float32)
            table = batch.shared[key] = ops.rope_table(batch.positions, self.inv_freq, out=out)
        return table

    def encode(self, q, k, positions, nh: int, nkv: int, d: int) -> None:
        """(A mixer that takes ``step_table`` does not come here.)"""
        table = ops.rope_table(positions, self.inv_freq)
        ops.rope_kv_store(q, None, None, table, None, None, None, nh, nkv, d)
        ops.rope_kv_store(k, None, None, table, None, None, None, nkv, nkv, d)


@register_position_encoding("rope_pairs")
class RopePairs(PositionEncoding):
    """Rotary encoding over neighbouring pairs: dims (2i, 2i + 1) of the first R = ``rotary_dim`` dims of each head
    turn by pos * theta^(-2i/R): (u, v) -> (u cos a - v sin a, v cos a + u sin a); the rest passes.
    params: head_dim, theta, rotary_dim (default head_dim).

    ``pair_table(batch)`` hands the step's (cos, sin) [n, R/2, 2] to mixers whose kernels turn pairs themselves;
    ``step_table`` stays None, because mixers read that table as one of split halves."""

    graph_safe = True
    tape_safe = True

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.head_dim = int(spec.params["head_dim"])
        self.rotary_dim = int(spec.params.get("rotary_dim", self.head_dim))
        self.theta = float(spec.params["theta"])
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rope_pairs: rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        if not self.theta > 0:
            raise ValueError("rope_pairs: theta must be positive")
        # the frequencies in double precision, rounded once
        i = np.arange(self.rotary_dim // 2, dtype=np.float64)
        self.inv_freq = torch.from_numpy(np.power(self.theta, -2.0 * i / self.rotary_dim).astype(np.float32)).to(rt.device)

    def pair_table(self, batch):
        key = ("rope_pairs", self.rotary_dim, self.theta)
        table = batch.shared.get(key)
        if table is None:
            out = self.rt.buffer(f"rope_pairs_table_{self.rotary_dim}_{self.theta!r}",
                                 (batch.num_tokens, self.rotary_dim // 2, 2), torch.float32)
            table = batch.shared[key] = ops.rope_table(batch.positions, self.inv_freq, out=out)
        return table

    def encode(self, q, k, positions, nh: int, nkv: int, d: int) -> None:
        table = ops.rope_table(positions, self.inv_freq)
        ops.rope_pairs(q, table, nh, d)
        ops.rope_pairs(k, table, nkv, d)


@register_position_encoding("none")
class NoPosition(PositionEncoding):
    """No encoding: keys and values are stored as they are."""

    graph_safe = True
    tape_safe = True

    def step_table(self, batch):
        return "none"

    def encode(self, q, k, positions, nh: int, nkv: int, d: int) -> None:
        pass
