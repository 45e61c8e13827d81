"""Rotary position encoding part.  Reference: ``jllm/model/common.py:51-66``.

``inv_freq[i] = theta ** (-2 i / dim)`` for i < dim/2, angle = position * inv_freq in
float; the pair (i, i + dim/2) of a head vector (half-split pairing, the reference's
``_rotate_half``) turns by its angle.  ``rotary_dim`` (default: the whole head) and
``interleaved`` pairing (2i, 2i+1) are parameters; elements past ``rotary_dim`` pass
through.  Cosines and sines of a step's positions are computed once per step, in float,
and shared by every layer with the same constants; the rotation itself runs inside the
attention-input kernel, which takes that table and this part's flags.
"""
from __future__ import annotations

import math

import torch

from ..ops import kernels as K
from .spec import register_part


class RotaryEncoding:
    replayable = True      # the table is computed on the device from the step's positions

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None, interleaved: bool = False,
                 rescale: dict | None = None, by_wavelength: dict | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        self.interleaved = bool(interleaved)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most the head size {self.head_dim}")
        # frequencies rescaled for contexts longer than the ``original`` one (YaRN): see ``inverse_frequencies``
        self.rescale = dict(rescale) if rescale else None
        self.amplitude = 0.1 * math.log(float(self.rescale["factor"])) + 1.0 if self.rescale else 1.0
        # frequencies slowed down by wavelength (the Llama 3.1 rule): see ``inverse_frequencies``
        self.by_wavelength = dict(by_wavelength) if by_wavelength else None
        if self.rescale and self.by_wavelength:
            raise ValueError("one rule for the frequencies, not two")
        self.inv_freq = None

    def tensors(self) -> dict:
        return {}

    def inverse_frequencies(self) -> torch.Tensor:
        """float32 table of rotary_dim/2 entries, computed as the reference does."""
        d = self.rotary_dim
        if self.by_wavelength is not None:
            # ``by_wavelength`` = {factor, low, high, original}: a pair whose wavelength 2 pi / f is below original / high
            # keeps f, one above original / low turns ``factor`` times slower, and between the two f is blended with
            # f / factor by s = (original / wavelength - low) / (high - low).  Computed in double, rounded once.
            r = {k: float(v) for k, v in self.by_wavelength.items()}
            f = self.theta ** (-2.0 * torch.arange(d // 2, dtype=torch.float64) / d)
            wave = 2 * math.pi / f
            s = (r["original"] / wave - r["low"]) / (r["high"] - r["low"])
            out = torch.where(wave < r["original"] / r["high"], f,
                              torch.where(wave > r["original"] / r["low"], f / r["factor"], (1 - s) * f / r["factor"] + s * f))
            return out.to(torch.float32)
        if self.rescale is None:
            return 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        # With ``rescale`` = {factor, original, fast, slow}: a pair that makes more than ``fast`` turns over
        # the original context keeps its frequency, one that makes fewer than ``slow`` turns is slowed down
        # by ``factor``, and the pairs between are blended linearly by their index; cos and sin are then
        # scaled by ``amplitude`` = 0.1 ln(factor) + 1.  Computed in double, rounded once.
        r = self.rescale
        i = torch.arange(d // 2, dtype=torch.float64)
        f = self.theta ** (-2.0 * i / d)

        def pair_with_turns(t: float) -> float:
            return d * math.log(float(r["original"]) / (2 * math.pi * t)) / (2 * math.log(self.theta))

        lo = max(math.floor(pair_with_turns(float(r["fast"]))), 0)
        hi = min(math.ceil(pair_with_turns(float(r["slow"]))), d - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        return (f / float(r["factor"]) * ramp + f * (1 - ramp)).to(torch.float32)

    def bind(self, tensors: dict, dtype: torch.dtype, device=None) -> None:
        self.inv_freq = self.inverse_frequencies().to(device or "cuda").contiguous()

    def as_rotation(self):
        """(rotary_dim, interleaved): this encoding is a rotation of q and k by position, which the
        mixer's own kernel applies from ``rotation_table``.  A position part that asks nothing of
        the mixer's kernels answers None."""
        return self.rotary_dim, self.interleaved

    def rotation_table(self, ctx):
        """Float cos/sin table of the step's positions for the attention-input kernel."""
        key = ("rope_table", self.theta, self.rotary_dim, tuple(sorted(self.rescale.items())) if self.rescale else None,
               tuple(sorted(self.by_wavelength.items())) if self.by_wavelength else None)
        table = ctx.extras.get(key)
        if table is None:
            if self.rescale is None:
                table = K.rope_table(ctx.positions, self.inv_freq)
            else:
                table = K.rope_table_amp(ctx.positions, self.inv_freq, self.amplitude)
            ctx.extras[key] = table
        return table


register_part("position", "rotary", RotaryEncoding)
