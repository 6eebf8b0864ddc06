"""Split-half rotary position encoding.

pair i in [0, rot/2): f_i = theta^(-2i/rot), phi = pos * f_i,
(x[i], x[i+rot/2]) <- (x[i]cos(phi) - x[i+rot/2]sin(phi), x[i]sin(phi) + x[i+rot/2]cos(phi)),
in 32-bit (crates/kernels-hip/src/kernels/rope_neox_partial_f16.cu:37-52).  The rotation
itself runs inside the mixer's rotate-and-store kernel; this part only carries its
constants."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import POSITION_ENCODINGS, PositionEncoding


@POSITION_ENCODINGS.register("rope_neox")
class RotaryNeoX(PositionEncoding):
    replayable = True

    def __init__(self, head_dim: int, theta: float, rotated_dims: int | None = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotated_dims = head_dim if rotated_dims is None else rotated_dims
        if self.rotated_dims % 2 or not 0 < self.rotated_dims <= head_dim:
            raise ValueError(f"rotated dims {self.rotated_dims} must be even and within the head size {head_dim}")

    def rotary_parameters(self):
        return self.rotated_dims, self.theta

    def inverse_frequencies(self):
        """``None``: the ladder ``theta^(-2 i / rotated_dims)``.  A subclass with another ladder (scaled,
        interpolated, cut) returns its ``rotated_dims / 2`` frequencies (floats, made in double) and
        may set ``magnitude``, a factor on every cosine and sine; everything else stays: the table is
        made from them, and the kernels that rotate read the table."""
        return None

    magnitude = 1.0

    def bind(self, weights, rt):
        self.rt = rt
        freqs = self.inverse_frequencies()
        self._ladder = None
        if freqs is not None:
            if len(freqs) != self.rotated_dims // 2:
                raise ValueError(f"{len(freqs)} frequencies for {self.rotated_dims} rotated dims")
            self._ladder = torch.tensor([float(f) for f in freqs], dtype=torch.float64, device=rt.device)
            self._ladder_key = tuple(float(f) for f in freqs)

    def rotary_table(self, rt, step):
        """The angles depend on the positions only: their cosines and sines are made once per
        forward pass and shared by all layers with the same constants."""
        ladder = getattr(self, "_ladder", None)
        key = ("rope_neox", self.rotated_dims, self.theta if ladder is None else self._ladder_key, self.magnitude)
        table = step.scratch.get(key)
        if table is None:
            half = self.rotated_dims // 2
            name = f"rope_table_{self.rotated_dims}_{self.theta}" if ladder is None else f"rope_table_{hash(key)}"
            table = rt.buffer(name, step.n_tokens, 2 * half, torch.float32)
            table = table.view(step.n_tokens, half, 2)
            if ladder is None:
                ops.rope_table(step.positions, self.rotated_dims, self.theta, table)
            else:
                ops.rope_table_ladder(step.positions, self.rotated_dims, ladder, table, self.magnitude)
            step.scratch[key] = table
        return table


@POSITION_ENCODINGS.register("none")
class NoPositionEncoding(PositionEncoding):
    replayable = True

    def __init__(self, **_):
        pass

    def rotary_parameters(self):
        return 0, 1.0


@POSITION_ENCODINGS.register("rope_interleaved")
class RotaryInterleaved(RotaryNeoX):
    """The same angles with the other pairing: dimension 2i turns with dimension 2i + 1.  The fused
    rotate-and-store kernels pair split halves, so this encoding offers its table and its ``layout``
    to mixers whose kernels read both."""
    layout = "interleaved"

    def rotary_parameters(self):
        return None


RotaryNeoX.layout = "half"


def blended_frequencies(rotated_dims: int, theta: float, factor: float, original: int, fast: float, slow: float):
    """A ladder of frequencies stretched for contexts beyond ``original`` positions: a dimension whose wave
    makes fewer than ``slow`` turns over ``original`` positions has its frequency divided by ``factor``, one
    that makes more than ``fast`` turns keeps it, and those between are mixed linearly in the dimension's
    index.  With ``turn(n) = dims * ln(original / (2 pi n)) / (2 ln theta)`` the (fractional) index whose
    wave makes n turns: lo = max(floor(turn(fast)), 0), hi = min(ceil(turn(slow)), dims - 1),
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), f_i' = f_i / factor * ramp_i + f_i (1 - ramp_i).
    Returns the frequencies and the factor 0.1 ln(factor) + 1 that goes on every cosine and sine."""
    import math
    def turn(n):
        return rotated_dims * math.log(original / (2.0 * math.pi * n)) / (2.0 * math.log(theta))
    lo = max(math.floor(turn(fast)), 0)
    hi = min(math.ceil(turn(slow)), rotated_dims - 1)
    out = []
    for i in range(rotated_dims // 2):
        f = theta ** (-2.0 * i / rotated_dims)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


@POSITION_ENCODINGS.register("rope_blended")
class RotaryBlended(RotaryNeoX):
    """Rotation with the stretched ladder of ``blended_frequencies``; ``layout``: ``half`` (split halves, which
    the fused rotate-and-store kernels take too) or ``interleaved``."""

    def __init__(self, head_dim: int, theta: float, factor: float, original: int, fast: float, slow: float,
                 rotated_dims: int | None = None, layout: str = "half"):
        super().__init__(head_dim, theta, rotated_dims)
        if layout not in ("half", "interleaved"):
            raise ValueError(f"rope_blended: layout must be 'half' or 'interleaved', got {layout!r}")
        self.layout = layout
        self._freqs, self.magnitude = blended_frequencies(self.rotated_dims, self.theta, float(factor), int(original),
                                                           float(fast), float(slow))

    def inverse_frequencies(self):
        return self._freqs

    def rotary_parameters(self):
        return super().rotary_parameters() if self.layout == "half" else None
