"""Rotary position encoding: the inverse frequencies, with the llama3 scaling of long wavelengths.

Only the frequencies and the form of the rotation live here (which elements make a pair, a factor on cosine and
sine); the rotation itself is fused into the kernels that write keys and values to the cache (``kernels.ops.rope_kv_write``
and the q/k/v products' epilogues, all through the one device function of ``csrc/rope.h``), which form
angle = position * inv_freq and its cosine and sine in 32-bit.  Reference: model/llama.py:98-118 (frequencies),
:133-136 (angles), :150-158 (pairing of element j with j + d/2).

A position encoding of another kind that the attention part can apply is an object with ``inv_freq`` (float32 on the
device, rotary_dim / 2 values), ``rotary_dim``, ``max_positions`` and optionally ``interleaved`` and ``factor``.
"""

from __future__ import annotations

import math

import torch

from .registry import register


def inverse_frequencies(rotary_dim: int, theta: float, scaling) -> torch.Tensor:
    """float32 [rotary_dim / 2], computed on the CPU as the reference does (model/llama.py:100-102)."""
    exponent = torch.arange(0, rotary_dim, 2, dtype=torch.int64, device="cpu").to(torch.float32) / rotary_dim
    inv = 1.0 / (theta ** exponent)
    if scaling is None:
        return inv
    factor, low, high, original = scaling
    wavelen = 2 * math.pi / inv
    long_wave, short_wave = original / low, original / high
    scaled = torch.where(wavelen > long_wave, inv / factor, inv)
    t = (original / wavelen - low) / (high - low)
    between = (wavelen >= short_wave) & (wavelen <= long_wave)
    return torch.where(between, (1 - t) * scaled / factor + t * scaled, scaled)


def yarn_frequencies(rotary_dim: int, theta: float, yarn) -> tuple[torch.Tensor, float]:
    """-> (float32 [rotary_dim / 2], factor on cosine and sine) for yarn = (factor, original, fast, slow): pairs whose
    wavelength is long against ``original`` turn ``factor`` times slower, short ones as they are, a linear ramp between
    (see ``config.spec.RopeSpec``).  Formed in 64-bit, then rounded once."""
    factor, original, fast, slow = (float(v) for v in yarn)
    j = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = theta ** (-2.0 * j / rotary_dim)
    at = lambda t: rotary_dim * math.log(original / (2 * math.pi * t)) / (2 * math.log(theta))
    lo = max(math.floor(at(fast)), 0)
    hi = min(math.ceil(at(slow)), rotary_dim - 1)
    ramp = ((j - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).to(torch.float32), 0.1 * math.log(factor) + 1.0


class Rope:
    graph_safe = True

    def __init__(self, spec, prefix: str = "") -> None:
        if spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim={spec.rotary_dim} must be even")
        self.spec = spec
        self.rotary_dim = spec.rotary_dim
        self.max_positions = spec.max_positions
        self.interleaved, self.factor = bool(spec.interleaved), float(spec.cos_sin_factor)
        self.inv_freq: torch.Tensor | None = None
        yarn = getattr(spec, "yarn", None)
        if yarn is not None:
            if spec.scaling is not None:
                raise ValueError("a rotation has one frequency scaling, not two")
            self._yarn_freq, mult = yarn_frequencies(spec.rotary_dim, spec.theta, yarn)
            self.factor *= mult

    def wanted(self) -> dict:
        return {}

    def load(self, get, dtype, device) -> None:
        if getattr(self.spec, "yarn", None) is not None:
            self.inv_freq = self._yarn_freq.to(device)
        else:
            self.inv_freq = inverse_frequencies(self.spec.rotary_dim, self.spec.theta, self.spec.scaling).to(device)


class NoPosition:
    """Keys and queries are left as they are."""

    graph_safe = True
    rotary_dim = 0
    max_positions = None
    interleaved, factor = False, 1.0

    def __init__(self, spec, prefix: str = "") -> None:
        self.inv_freq = None

    def wanted(self) -> dict:
        return {}

    def load(self, get, dtype, device) -> None:
        self.inv_freq = torch.zeros(1, dtype=torch.float32, device=device)


register("position", "rope", Rope)
register("position", "none", NoPosition)
