"""Rotary position encoding: the table of inverse frequencies.

f_i = theta^(-2i/d) for i < d/2; the angle of position p is p * f_i and pairs are
half-split, (x[i], x[i + d/2]) (infernum/src/rope.rs:19-30,
infernum-cuda/kernels/rope.cu:25-41).  The rotation itself runs in the kernel
that also writes keys and values to their pages; this part owns the
frequencies only, which is all that differs between encodings of this family.

``llama3`` scaling is not in the reference's Llama path.  It has the form of
the reference's YaRN bands (infernum/src/rope.rs:91-120) with the band edges
taken from the configuration: with wavelength L = 2 pi / f and the original
context n, L < n/high keeps f, L > n/low gives f/factor, and between them
f' = (1-r) f/factor + r f with r = (n/L - low) / (high - low).  There is no
magnitude correction.

``yarn`` scaling (keys ``factor``, ``original``, ``fast``, ``slow``) blends by the pair's index instead of its
wavelength: with dim(t) = rot ln(original / (2 pi t)) / (2 ln theta), the index at which a pair makes t turns over the
original context, lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), rot - 1) and
r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at f_i / factor * r_i + f_i (1 - r_i); sine and cosine
are both multiplied by ``magnitude`` = 0.1 ln(factor) + 1 (the reference's YaRN, infernum/src/rope.rs:91-120, has the
same bands and correction).  ``pairing`` "neighbours" pairs value 2i with value 2i + 1 in place of i with i + rot/2.
``linear`` scaling (key ``factor``) divides every frequency by the factor.

Frequencies are formed and kept in float64; the rotation kernel forms the angle
position * frequency in float64 too and brings it into [-pi, pi] before it takes
the fp32 sine and cosine, so that the angle is as good at position 100,000 as at
position 1 (a table of fp32 frequencies, which a position encoding may also give,
is multiplied in fp32: off by up to position * 2^-24 rad).
"""
from __future__ import annotations

import math
from typing import Any, Mapping, Optional

import torch

from .base import PositionEncoding, Runtime, register_part


def rope_inverse_frequencies(rotary_dim: int, theta: float, scaling: Optional[Mapping[str, Any]] = None) -> torch.Tensor:
    """float64 [rotary_dim / 2] on the CPU."""
    if rotary_dim <= 0 or rotary_dim % 2:
        raise ValueError(f"rotary size must be even and positive, got {rotary_dim}")
    half = rotary_dim // 2
    freqs = []
    for i in range(half):
        f = float(theta) ** (-2.0 * i / rotary_dim)
        if scaling is not None:
            kind = scaling.get("rope_type")
            if kind == "yarn":
                freqs.append(f)
                continue
            if kind == "linear":            # every frequency divided by the factor: positions counted in 1/factor steps
                freqs.append(f / float(scaling["factor"]))
                continue
            if kind != "llama3":
                raise ValueError(f"rope scaling of type {kind!r} is not supported")
            factor = float(scaling["factor"])
            low = float(scaling["low_freq_factor"])
            high = float(scaling["high_freq_factor"])
            n = float(scaling["original_max_position_embeddings"])
            wavelen = 2.0 * math.pi / f
            if wavelen < n / high:
                pass
            elif wavelen > n / low:
                f = f / factor
            else:
                r = (n / wavelen - low) / (high - low)
                f = (1.0 - r) * f / factor + r * f
        freqs.append(f)
    if scaling is not None and scaling.get("rope_type") == "yarn":
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def index_of_turns(turns: float) -> float:
            return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(theta)))
        lo = max(math.floor(index_of_turns(float(scaling["fast"]))), 0)
        hi = min(math.ceil(index_of_turns(float(scaling["slow"]))), rotary_dim - 1)
        for i in range(half):
            r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            freqs[i] = freqs[i] / factor * r + freqs[i] * (1.0 - r)
    return torch.tensor(freqs, dtype=torch.float64)


def rope_magnitude(scaling: Optional[Mapping[str, Any]]) -> float:
    """The factor on sine and cosine: 0.1 ln(factor) + 1 under ``yarn`` scaling, 1 otherwise."""
    if scaling is not None and scaling.get("rope_type") == "yarn":
        return 0.1 * math.log(float(scaling["factor"])) + 1.0
    return 1.0


class RotaryEmbedding(PositionEncoding):
    """Half-split rotary encoding of the first ``rotary_dim`` values of a head."""
    graph_safe = True

    def __init__(self, rt: Runtime, head_dim: int, theta: float, scaling: Optional[Mapping[str, Any]] = None,
                 rotary_dim: Optional[int] = None, pairing: str = "half"):
        super().__init__(rt)
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        if self.rotary_dim > self.head_dim:
            raise ValueError("rotary_dim larger than the head size")
        if pairing not in ("half", "neighbours"):
            raise ValueError(f"pairing {pairing!r}: 'half' or 'neighbours'")
        self.pairing = pairing
        self.magnitude = rope_magnitude(scaling)
        self.inv_freq = rope_inverse_frequencies(self.rotary_dim, theta, scaling).to(rt.device)

    def head_permutation(self) -> Optional[torch.Tensor]:
        """For kernels that pair value i with value i + rot/2: the order of a head's values that makes those pairs
        the neighbours' (kernels that take a pairing need none)."""
        if self.pairing == "half":
            return None
        r = self.rotary_dim
        return torch.tensor(list(range(0, r, 2)) + list(range(1, r, 2)) + list(range(r, self.head_dim)), dtype=torch.int64)


class NoPositionEncoding(PositionEncoding):
    """Queries and keys are used as they are."""
    graph_safe = True

    def __init__(self, rt: Runtime, **_: Any):
        super().__init__(rt)
        self.inv_freq = None
        self.rotary_dim = 0
        self.pairing, self.magnitude = "half", 1.0


register_part("position", "rope", RotaryEmbedding)
register_part("position", "none", NoPositionEncoding)
