"""Position encodings. GPT-2 adds a learned row per absolute position to the token embedding
(src/levanter/models/gpt2.py:291-296,302-308) and has nothing inside attention."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .base import BuildEnv, PositionEncoding, StepContext
from .registry import POSITION_ENCODINGS
from .spec import PartSpec


@POSITION_ENCODINGS.register("learned_absolute")
class LearnedAbsolutePosition(PositionEncoding):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.max_positions = int(spec.params["n_positions"])
        self.table = tensors["table"].to(env.device, env.dtype).contiguous()

    def embedding_table(self) -> Optional[torch.Tensor]:
        return self.table


@POSITION_ENCODINGS.register("none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)


def rotary_frequencies(dims: int, base: float, scaling: Optional[dict] = None) -> List[float]:
    """The angle per position of each of the ``dims / 2`` pairs: ``base^(-2i/dims)``. ``scaling`` (``factor``, ``low``,
    ``high``, ``original``) stretches the slow pairs for longer contexts than the ``original`` one: a pair whose wavelength
    ``2 pi / f`` is shorter than ``original / high`` keeps its frequency, one longer than ``original / low`` turns
    ``factor`` times slower, and between the two the frequency goes linearly, in ``original / wavelength``, from the one to
    the other. A ``scaling`` with the keys ``fast`` and ``slow`` is the other rule, ``ramp_frequencies``."""
    if scaling and "fast" in scaling:
        return ramp_frequencies(dims, base, scaling)
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                f = f / factor
            elif wavelength >= original / high:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def ramp_frequencies(dims: int, base: float, scaling: dict) -> List[float]:
    """``base^(-2i/dims)`` stretched by pair index (``factor``, ``original``, ``fast``, ``slow``): with
    ``index(t) = dims ln(original / (2 pi t)) / (2 ln base)`` the index of the pair that makes ``t`` turns over the ``original``
    length, pairs up to ``lo = max(floor(index(fast)), 0)`` keep their frequency, pairs from ``hi = min(ceil(index(slow)), dims - 1)``
    on turn ``factor`` times slower, and between them the two frequencies are mixed linearly in the index."""
    factor, original, fast, slow = (float(scaling[k]) for k in ("factor", "original", "fast", "slow"))

    def index(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

    lo = max(math.floor(index(fast)), 0)
    hi = min(math.ceil(index(slow)), dims - 1)
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out


@POSITION_ENCODINGS.register("rotary_pairs")
class RotaryPairs(PositionEncoding):
    """Rotates neighbouring dimensions (2i, 2i+1) of every query and key head by ``position * f_i`` (the interleaved
    layout), on the first ``dims`` dimensions of a head; the rest pass unchanged. params: ``head_dim`` (the size of a head as
    the mixer stores it), ``dims``, ``base``, ``scaling`` (see ``rotary_frequencies``; None: none), ``magnitude`` (a factor on
    cosine and sine alike; 1 by default). Angles are 32-bit."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.head_dim, self.dims = int(p["head_dim"]), int(p["dims"])
        if self.dims % 2 or not 0 <= self.dims <= self.head_dim:
            raise ValueError(f"rotary_pairs: {self.dims} rotated dimensions must be even and fit a head of {self.head_dim}")
        self.freqs = torch.tensor(rotary_frequencies(self.dims, p["base"], p.get("scaling")), dtype=torch.float64).to(torch.float32).to(env.device)
        self.magnitude = float(p.get("magnitude", 1.0))

    def rotate(self, q: torch.Tensor, k: torch.Tensor, ctx: StepContext) -> None:
        if self.dims:
            if self.magnitude == 1.0:
                ctx.kernels.rotary_pairs(q, k, self.head_dim, self.freqs, ctx.attention.positions)
            else:
                ctx.kernels.rotary_pairs(q, k, self.head_dim, self.freqs, ctx.attention.positions, magnitude=self.magnitude)
