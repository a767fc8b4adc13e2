"""Rotary position encoding: the table of angles per pair and how pairs are formed.

``freq_i = 1 / theta^(2i / rotary_dim)`` evaluated in float32 as the reference does
(``1.0f / powf(base, 2.0f * i / head_dim)``, /root/reference/src/engine/tq_ops.c:1418-1448); the angle of
pair i at position p is ``p * freq_i`` in float32.  ``pairing`` says which two dimensions form pair i:
``"half"`` pairs (i, i + rotary_dim/2) (/root/reference/src/engine/tq_transformer.c:1263-1289), the layout of
un-permuted checkpoints (/root/reference/docs/supported_models.md:99-108); ``"interleaved"`` pairs
(2i, 2i+1) as ``tq_rope`` does.  Dimensions from ``rotary_dim`` on are not rotated.

A mixer asks a position part for three things only: ``table(device)`` (float32 [rotary_dim/2] angles
per position step), ``pairing_code`` and ``rotary_dim``.  Another encoding that rotates pairs (scaled,
partial, with per-pair factors) is another table.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from .base import Part, register_part

PAIRINGS = {"half": 0, "interleaved": 1}


@register_part("position", "rope")
class RotaryEncoding(Part):
    graph_safe = True
    amplitude = 1.0          # a factor on every sine and cosine (other encodings scale them)

    def __init__(self, head_dim: int, rotary_dim: int, theta: float, pairing: str = "half", double_table: bool = False):
        """``double_table``: the frequencies are worked out in double precision and rounded once, instead of in float32."""
        self.double_table = double_table
        if pairing not in PAIRINGS:
            raise ValueError(f"unknown pairing {pairing!r}; known: {sorted(PAIRINGS)}")
        if rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and at most head_dim {head_dim}")
        self.head_dim, self.rotary_dim, self.theta, self.pairing = head_dim, rotary_dim, theta, pairing
        self._table = None

    @property
    def pairing_code(self) -> int:
        return PAIRINGS[self.pairing]

    def frequencies(self) -> np.ndarray:
        if self.double_table:
            i = np.arange(self.rotary_dim // 2, dtype=np.float64)
            return np.power(float(self.theta), -2.0 * i / max(self.rotary_dim, 1)).astype(np.float32)
        i = np.arange(self.rotary_dim // 2, dtype=np.float32)
        expo = (np.float32(2.0) * i) / np.float32(self.rotary_dim)
        return (np.float32(1.0) / np.power(np.float32(self.theta), expo, dtype=np.float32)).astype(np.float32)

    def table(self, device) -> torch.Tensor:
        if self._table is None or self._table.device != torch.device(device):
            self._table = torch.from_numpy(self.frequencies()).to(device)
        return self._table

    def prepare(self, device, act):
        self.table(device)


@register_part("position", "none")
class NoRotation(Part):
    """No rotation of queries and keys: for models whose positions enter elsewhere (a learned vector added to the
    embedding, a bias on the scores).  A mixer sees an empty table and a rotary width of 0."""
    graph_safe = True
    pairing_code = 0
    rotary_dim = 0
    amplitude = 1.0

    def __init__(self):
        self._table = None

    def table(self, device) -> torch.Tensor:
        if self._table is None or self._table.device != torch.device(device):
            self._table = torch.zeros((1,), dtype=torch.float32, device=device)[:0]
        return self._table

    def prepare(self, device, act):
        self.table(device)


@register_part("position", "llama3_rope")
class Llama3RotaryEncoding(RotaryEncoding):
    """Rotary encoding whose slow pairs are slowed down further, by wavelength, for sequences longer than the ``original``
    length.  With f_i = theta^(-2i / rotary_dim) and the pair's wavelength l = 2 pi / f_i: f_i stays where
    l < original / high; it becomes f_i / factor where l > original / low; in between, with
    s = (original / l - low) / (high - low), it becomes (1 - s) f_i / factor + s f_i.  The table is worked out in double
    precision and rounded once; nothing else of the rotation changes."""

    def __init__(self, head_dim: int, rotary_dim: int, theta: float, factor: float, original: float, low: float, high: float,
                 pairing: str = "half"):
        super().__init__(head_dim, rotary_dim, theta, pairing)
        if not (factor > 0 and original > 0 and low > 0 and high > low and theta > 0):
            raise ValueError("the stretched rotation needs positive factor, theta, original and low, and high above low")
        self.factor, self.original, self.low, self.high = float(factor), float(original), float(low), float(high)

    def frequencies(self) -> np.ndarray:
        i = np.arange(self.rotary_dim // 2, dtype=np.float64)
        f = np.power(float(self.theta), -2.0 * i / max(self.rotary_dim, 1))
        length = 2.0 * math.pi / f
        s = (self.original / length - self.low) / (self.high - self.low)
        out = np.where(length < self.original / self.high, f,
                       np.where(length > self.original / self.low, f / self.factor, (1.0 - s) * f / self.factor + s * f))
        return out.astype(np.float32)


@register_part("position", "yarn_rope")
class YarnRotaryEncoding(RotaryEncoding):
    """Rotary encoding whose slow pairs are stretched for sequences longer than the ``original`` length (YaRN).

    With f_i = theta^(-2i / rotary_dim) and where(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta), the (fractional)
    pair that makes t turns over the original length: lo = max(floor(where(fast)), 0), hi = min(ceil(where(slow)),
    rotary_dim - 1), ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1); pair i turns at
    f_i / factor * ramp_i + f_i (1 - ramp_i), and every sine and cosine is multiplied by ``amplitude`` =
    0.1 ln(factor) + 1.  The table is worked out in double precision and rounded once; a mixer multiplies positions by
    it in float32 and asks for ``amplitude`` beside ``table``, ``pairing_code`` and ``rotary_dim``."""

    def __init__(self, head_dim: int, rotary_dim: int, theta: float, factor: float, original: float, fast: float,
                 slow: float, pairing: str = "half"):
        super().__init__(head_dim, rotary_dim, theta, pairing)
        if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and theta > 0 and theta != 1.0):
            raise ValueError("YaRN needs a theta other than 1 and positive factor, theta, original, fast and slow")
        self.factor, self.original, self.fast, self.slow = float(factor), float(original), float(fast), float(slow)
        self.amplitude = 0.1 * math.log(self.factor) + 1.0

    def _where(self, turns: float) -> float:
        return self.rotary_dim * math.log(self.original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

    def frequencies(self) -> np.ndarray:
        n = self.rotary_dim // 2
        i = np.arange(n, dtype=np.float64)
        f = np.power(float(self.theta), -2.0 * i / max(self.rotary_dim, 1))
        lo = max(math.floor(self._where(self.fast)), 0)
        hi = min(math.ceil(self._where(self.slow)), self.rotary_dim - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return (f / self.factor * ramp + f * (1.0 - ramp)).astype(np.float32)
