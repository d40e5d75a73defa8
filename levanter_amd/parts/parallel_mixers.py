"""Two mixers side by side: both read the layer's normed input, and the layer adds ``left_scale * left + right_scale *
right``. The two keep what they need in one cache unit (pages for an attention, a state slot for a recurrence).

Where both offer ``proj`` / ``attend`` / ``out`` their first products become one (the weights' rows side by side) and their
last products one: each branch multiplies what it hands to ``out`` by its scale (in 32-bit, before it is rounded to the
compute dtype), and the one product over ``[left | right]`` columns is the weighted sum.

With ``branch_norm_eps`` each branch's result passes an RMS norm over the model's width with a weight of its own
(``left_norm.weight``, ``right_norm.weight``) before the weighted sum: the two last products then stay apart (each into a 32-bit
tensor of its own) and one row kernel norms and adds them.
"""
from __future__ import annotations

import inspect
from typing import Dict, Optional

import torch

from levanter_amd.cache.requirements import Combined
from .base import BuildEnv, CacheUnitView, Mixer, StepContext
from .embedding import tensors_of_nested
from .linear import Linear
from .registry import MIXERS, part_class
from .spec import PartSpec


@MIXERS.register("parallel_mixers")
class ParallelMixers(Mixer):
    """params: ``left``, ``right`` (descriptions of mixers that take an ``out_scale``), ``left_scale``, ``right_scale``, ``branch_norm_eps``
    (None: the branches are added as they are; else with the tensors ``left_norm.weight`` and ``right_norm.weight`` ``[dim]``)."""

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.branches = []
        self.branch_norm_eps = p.get("branch_norm_eps")
        self.scales = [float(p.get(f"{side}_scale", 1.0)) for side in ("left", "right")]
        for side in ("left", "right"):
            sub: PartSpec = p[side]
            # with a norm behind each branch the branch's weight is applied behind the norm, not to what the branch hands over
            scale = 1.0 if self.branch_norm_eps is not None else float(p.get(f"{side}_scale", 1.0))
            sub = PartSpec(sub.kind, {**sub.params, "out_scale": scale}, sub.tensors, sub.family)
            self.branches.append(part_class(sub.kind, sub.family or "mixer")(sub, tensors_of_nested(side, tensors), env))
        for b in self.branches:
            if not all(hasattr(b, a) for a in ("proj", "attend", "out")):
                raise ValueError(f"parallel_mixers: the mixer {b.kind!r} does not offer proj / attend / out")
        self.graph_safe = all(bool(b.graph_safe) for b in self.branches)
        self.wants_input = ["h" in inspect.signature(b.attend).parameters for b in self.branches]
        left, right = self.branches
        if left.proj.n_out % 8 or left.out.n_in % 8 or left.proj.weight.dtype != right.proj.weight.dtype:
            raise ValueError("parallel_mixers: the left mixer's products must be multiples of 8 wide (the right one's columns follow them)")
        self.proj_cols = [b.proj.n_out for b in self.branches]
        self.out_cols = [b.out.n_in for b in self.branches]

        def cat_bias(a: Optional[torch.Tensor], b: Optional[torch.Tensor], na: int, nb: int):
            if a is None and b is None:
                return None
            dev = (a if a is not None else b).device
            return torch.cat([a if a is not None else torch.zeros(na, device=dev), b if b is not None else torch.zeros(nb, device=dev)])

        self.proj = Linear(torch.cat([left.proj.weight, right.proj.weight], 0), cat_bias(left.proj.bias, right.proj.bias, *self.proj_cols), "out_in", env)
        if self.branch_norm_eps is not None:
            self.branch_norm_eps = float(self.branch_norm_eps)
            self.norm_weights = [tensors[f"{side}_norm.weight"].to(env.device, torch.float32).contiguous() for side in ("left", "right")]
            self.outs = [b.out for b in self.branches]
            if any(w.numel() != o.n_out for w, o in zip(self.norm_weights, self.outs)) or left.out.n_out != right.out.n_out:
                raise ValueError("parallel_mixers: the branches' norm weights must be as wide as the branches' results")
            self.out = None
            for b in self.branches:
                b.proj = None
            return
        out_bias = None if left.out.bias is None and right.out.bias is None else sum(b.out.bias for b in self.branches if b.out.bias is not None)
        self.out = Linear(torch.cat([left.out.weight, right.out.weight], 1), out_bias, "out_in", env)
        for b in self.branches:  # their own copies are not needed any more
            b.proj = b.out = None

    def cache_requirement(self):
        reqs = tuple(r for r in (b.cache_requirement() for b in self.branches) if r is not None)
        return reqs[0] if len(reqs) == 1 else (Combined(reqs) if reqs else None)

    def _normed_sum(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        """``y`` = the weighted sum of the branches' results, each through its norm."""
        a = ctx.empty(h.shape[0], sum(self.out_cols))
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a, h=h)
        n_left = self.out_cols[0]
        left = self.outs[0](a[:, :n_left], ctx, out_dtype=torch.float32)
        self.outs[1](a[:, n_left:], ctx, out=y)
        ctx.kernels.norm_sum2(left, y, self.norm_weights[0], self.norm_weights[1], self.scales[0], self.scales[1], self.branch_norm_eps, y)

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        if self.branch_norm_eps is not None:
            y = torch.empty_like(x)
            self._normed_sum(h, y, ctx, unit, writes_cache)
            ctx.settle()
            x.add_(y)
            return
        a = ctx.empty(h.shape[0], self.out.n_in)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a, h=h)
        self.out(a, ctx, residual=x, final=True)

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        if self.branch_norm_eps is not None:
            self._normed_sum(h, y, ctx, unit, writes_cache)
            return
        a = ctx.empty(h.shape[0], self.out.n_in)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a, h=h)
        self.out(a, ctx, out=y, may_leave=True)

    def attend(self, p: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool, a: torch.Tensor, h: torch.Tensor = None) -> None:
        """``h``: the mixers' input, for a branch whose ``attend`` asks for it (products of its own beside ``proj``)."""
        pc, ac = 0, 0
        for b, n_p, n_a, wants_h in zip(self.branches, self.proj_cols, self.out_cols, self.wants_input):
            extra = {"h": h} if h is not None and wants_h else {}
            b.attend(p[:, pc:pc + n_p], ctx, unit, writes_cache, a[:, ac:ac + n_a], **extra)
            pc, ac = pc + n_p, ac + n_a
