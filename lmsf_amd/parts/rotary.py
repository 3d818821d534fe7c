"""Rotary position embedding.

Frequencies f_i = theta^(-2i/rot), angle = position * f_i, cos and sin kept as a float32 table
[max_positions, rot] = [cos | sin] (core/src/model_executor/layers/rotary_embedding.rs:46-66 builds
the same table, but with the base fixed to 10000 (:105), 4096 rows
(core/src/model_executor/models/llama/llama.rs:18) and cast to the model's dtype). The rotation
itself is done by the kernel that also writes the cache.

rope_scaling "llama3" changes each frequency by its wavelength L = 2 pi / f relative to the
original context length o: L < o / high_freq_factor keeps f, L > o / low_freq_factor gives
f / factor, in between (1 - s) f / factor + s f with s = (o / L - low) / (high - low).

rope_scaling "yarn" blends by the pair's index instead: with turn(t) = rot ln(o / (2 pi t)) / (2 ln theta) the index
at which a pair makes t turns over the original length o, lo = max(floor(turn(beta_fast)), 0),
hi = min(ceil(turn(beta_slow)), rot - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i gets
f_i / factor * ramp_i + f_i (1 - ramp_i); and cos and sin are both multiplied by 0.1 ln(factor) + 1
(``table_gain``), which the table carries.
"""
import math
from typing import Any, Callable, Mapping, Optional

import torch

from .base import PositionEncoding, Runtime, register_part


def inverse_frequencies(rotary_dim: int, theta: float, scaling: Optional[Mapping[str, Any]]) -> torch.Tensor:
    """float32 [rotary_dim / 2]."""
    exponent = torch.arange(0, rotary_dim, 2, dtype=torch.float32) / float(rotary_dim)
    inv = torch.reciprocal(torch.pow(torch.tensor(theta, dtype=torch.float32), exponent))
    kind = "default" if not scaling else scaling.get("rope_type", "default")
    if kind == "default":
        return inv
    if kind == "yarn":
        factor, orig = float(scaling["factor"]), float(scaling["original_max_position_embeddings"])

        def turn(t: float) -> float:
            return rotary_dim * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(theta))

        lo = max(math.floor(turn(float(scaling["beta_fast"]))), 0)
        hi = min(math.ceil(turn(float(scaling["beta_slow"]))), rotary_dim - 1)
        idx = torch.arange(rotary_dim // 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * idx / rotary_dim)
        ramp = torch.clamp((idx - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return (f / factor * ramp + f * (1.0 - ramp)).to(torch.float32)
    if kind != "llama3":
        raise ValueError("rotary scaling %r is not supported (default, llama3, yarn)" % kind)
    factor = float(scaling["factor"])
    low, high = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    f = inv.to(torch.float64)
    wavelength = 2.0 * math.pi / f
    smooth = (orig / wavelength - low) / (high - low)
    blended = (1.0 - smooth) * f / factor + smooth * f
    scaled = torch.where(wavelength < orig / high, f, torch.where(wavelength > orig / low, f / factor, blended))
    return scaled.to(torch.float32)


def table_gain(scaling: Optional[Mapping[str, Any]]) -> float:
    """What cos and sin are multiplied by: 0.1 ln(factor) + 1 under "yarn" scaling, else 1."""
    if scaling and scaling.get("rope_type") == "yarn":
        return 0.1 * math.log(float(scaling["factor"])) + 1.0
    return 1.0


@register_part("position", "rotary")
class RotaryEncoding(PositionEncoding):
    """style "neox" pairs (i, i + rot/2), "gptj" pairs (2i, 2i+1)
    (vllm/kernels/pos_encoding_kernels.cu:12-36)."""

    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, head_dim: int, theta: float, rotary_dim: Optional[int] = None,
                 scaling: Optional[Mapping[str, Any]] = None, style: str = "neox", angles: str = "float32"):
        super().__init__(prefix, rt)
        # "float64": frequencies, angles, cosines and sines are worked out in float64 and rounded once, into the
        # float32 table (unscaled frequencies only); "float32": in float32 throughout, as the reference does
        if angles not in ("float32", "float64") or (angles == "float64" and scaling):
            raise ValueError("rotary angles %r unknown (float32, float64 without scaling)" % angles)
        self.angles = angles
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim else self.head_dim
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim or self.rotary_dim <= 0:
            raise ValueError("rotary_dim %d must be even and within head_dim %d" % (self.rotary_dim, self.head_dim))
        if style not in ("neox", "gptj"):
            raise ValueError("rotary style %r unknown (neox, gptj)" % style)
        self.theta = float(theta)
        self.scaling = None if not scaling else dict(scaling)
        self.neox = style == "neox"
        self.table: Optional[torch.Tensor] = None

    def _key(self):
        sc = None if self.scaling is None else tuple(sorted(self.scaling.items()))
        return ("rotary_table", self.rotary_dim, self.theta, sc, self.rt.max_positions, self.angles)

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        key = self._key()
        if key not in self.rt.shared and self.angles == "float64":
            idx = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
            inv = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * idx / self.rotary_dim)
            angles = torch.arange(self.rt.max_positions, dtype=torch.float64)[:, None] * inv[None, :]
            table = torch.cat([torch.cos(angles), torch.sin(angles)], dim=1).to(torch.float32).contiguous()
            self.rt.shared[key] = table.to(self.rt.device)
        if key not in self.rt.shared:
            inv = inverse_frequencies(self.rotary_dim, self.theta, self.scaling)
            pos = torch.arange(self.rt.max_positions, dtype=torch.float32)
            angles = pos[:, None] * inv[None, :]
            table = torch.cat([torch.cos(angles), torch.sin(angles)], dim=1).contiguous()
            gain = table_gain(self.scaling)
            if gain != 1.0:
                table = table * gain
            self.rt.shared[key] = table.to(self.rt.device)
        self.table = self.rt.shared[key]

    def rotary_table(self):
        """(table float32 [max_positions, rot], rotary_dim, neox) for the fused rotate-and-store kernel."""
        return self.table, self.rotary_dim, self.neox

    def apply(self, qkv: torch.Tensor, nh: int, nkv: int, d: int, positions: torch.Tensor) -> None:
        self.rt.ops.rope_cache_write(qkv, nh, nkv, d, positions, self.table, self.rotary_dim, self.neox,
                                     None, None, None)
