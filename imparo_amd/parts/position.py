"""Position encodings. A position part owns a table of inverse frequencies
and says which dimensions make a pair (`interleaved` False: i with i +
rotary_dim/2; True: 2i with 2i + 1); the attention mixer hands both to the
fused norm+rotation kernel together with each token's absolute position.

NeoX rotation: dimension i pairs with i + rotary_dim/2, inv_i =
base^(-2i/rotary_dim), angle = position * inv_i
(/root/reference/crates/imparo-cpu/src/ops.rs:551-569). `wavelength_scaling`
(factor, low, high, original) rescales the table by wavelength; `precise`
takes the table in float64 before it is rounded to float32."""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from ..config.plan import PartSpec
from .registry import register_part


def scale_by_wavelength(inv_freq: np.ndarray, factor: float, low: float, high: float, original: float) -> np.ndarray:
    """Frequency scaling by wavelength, as Llama 3.1 stretches a context of `original` positions: a
    frequency whose wavelength 2 pi / f is shorter than original / high stays; one longer than
    original / low is divided by `factor`; between the two it is (1 - s) f / factor + s f with
    s = (original / wavelength - low) / (high - low)."""
    f = np.asarray(inv_freq, dtype=np.float64)
    wavelength = 2.0 * np.pi / f
    s = (original / wavelength - low) / (high - low) if high != low else np.ones_like(f)
    blended = (1.0 - s) * f / factor + s * f
    return np.where(wavelength < original / high, f, np.where(wavelength > original / low, f / factor, blended))


class RopeNeox:
    role = "position"
    interleaved = False

    def __init__(self, spec: PartSpec, device: torch.device):
        self.rotary_dim = int(spec["rotary_dim"])
        self.base = float(spec["base"])
        if self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {self.rotary_dim}")
        half = self.rotary_dim // 2
        scaling = spec.get("wavelength_scaling")
        if spec.get("precise") or scaling is not None:
            # the table in float64, rounded to float32 once at the end
            inv = np.power(np.float64(self.base), -2.0 * np.arange(half, dtype=np.float64) / self.rotary_dim)
            if scaling is not None:
                inv = scale_by_wavelength(inv, **{k: float(scaling[k]) for k in ("factor", "low", "high", "original")})
            inv = inv.astype(np.float32)
        else:
            i = np.arange(half, dtype=np.float32)
            expo = (np.float32(-2.0) * i / np.float32(self.rotary_dim)).astype(np.float32)
            inv = np.power(np.float32(self.base), expo).astype(np.float32)
        factors = spec.get("frequency_factors")
        if factors is not None:      # divides theta per pair
            inv = (inv / np.asarray(factors, dtype=np.float32)).astype(np.float32)
        self.inv_freq: Optional[torch.Tensor] = torch.from_numpy(inv).to(device)


class RopePairs(RopeNeox):
    """The same table with neighbouring dimensions as pairs: pair i is dims (2i, 2i + 1)."""
    interleaved = True


class NoPosition:
    """No rotation: keys are cached as the norm leaves them."""
    role = "position"

    interleaved = False

    def __init__(self, spec: PartSpec, device: torch.device):
        self.rotary_dim = 0
        self.inv_freq = None


register_part("position", "rope_neox", RopeNeox)
register_part("position", "rope_pairs", RopePairs)
register_part("position", "none", NoPosition)
