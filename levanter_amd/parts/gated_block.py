"""A layer whose sublayers stand between two norms and enter the residual stream through a gate, and the norm in groups it uses.

``gn(v, w)``: the vector in ``groups`` equal consecutive parts, each divided by its own sqrt(mean(part^2) + eps), the whole times
``w`` (one group: the plain RMS norm). A sublayer f with the input h = gn(x, w_pre) adds

    x <- x + mult * gn(f(h) * sigmoid(W_gate h + b_gate), w_post)

to the residual stream: its result is gated element by element by a function of its own input, normed again and scaled.
All of it but the gate's product is 32-bit and runs as one row kernel; the write of one sublayer is not launched by itself but
left pending and done by the pass that reads the stream next (the next sublayer's norm, the next layer's, or the norm before
the head), so a sublayer costs one row kernel.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from levanter_amd.kernels.library import PendingGatedNorm
from .base import Block, BuildEnv, CacheUnitView, Norm, Part, StepContext
from .linear import Linear
from .registry import BLOCKS, NORMS, STREAM_MIXES
from .spec import PartSpec


@NORMS.register("group_rmsnorm")
class GroupRmsNorm(Norm):
    """params: ``dim``, ``groups``, ``eps``; tensor ``weight`` ``[dim]``. Folds a pending gated write of the same grouping into
    its pass."""

    graph_safe = True
    folds_pending = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.dim, self.groups, self.eps = int(spec.params["dim"]), int(spec.params["groups"]), float(spec.params["eps"])
        if self.dim % self.groups:
            raise ValueError(f"group_rmsnorm: {self.dim} numbers do not split into {self.groups} equal groups")
        self.weight = tensors["weight"].to(env.device, torch.float32).contiguous()
        if self.weight.numel() != self.dim:
            raise ValueError(f"group_rmsnorm: the weight must have {self.dim} entries, got {self.weight.numel()}")

    def __call__(self, x: torch.Tensor, ctx: StepContext, rows: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.numel()
        out = ctx.empty(n, self.dim, out_dtype)
        pending = ctx.take_pending(x)
        if pending is not None and not (isinstance(pending, PendingGatedNorm) and pending.groups == self.groups and pending.eps == self.eps):
            ctx.kernels.finish(pending)
            pending = None
        ctx.kernels.group_norm_step(x, groups=self.groups, eps=self.eps, weight=self.weight, h_out=out, rows=rows, pending=pending)
        return out


@STREAM_MIXES.register("gated_post_norm")
class GatedPostNorm(Part):
    """How one sublayer's result enters the residual stream: ``x <- x + mult * gn(y * sigmoid(gate.weight h + gate.bias), weight)``.
    params: ``dim``, ``groups``, ``eps``, ``mult``, ``gate`` (False: no gate and no gate tensors). Tensors: ``weight`` ``[dim]``,
    ``gate.weight`` ``[dim, dim]``, ``gate.bias`` ``[dim]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim, self.groups, self.eps, self.mult = int(p["dim"]), int(p["groups"]), float(p["eps"]), float(p.get("mult", 1.0))
        self.weight = tensors["weight"].to(env.device, torch.float32).contiguous()
        self.gate = Linear(tensors["gate.weight"], tensors.get("gate.bias"), "out_in", env) if p.get("gate", True) else None
        if self.weight.numel() != self.dim or (self.gate is not None and (self.gate.n_in, self.gate.n_out) != (self.dim, self.dim)):
            raise ValueError("gated_post_norm: weights do not have the sizes of the description")

    def gate_of(self, h: torch.Tensor, ctx: StepContext) -> Optional[torch.Tensor]:
        """``gate.weight h + gate.bias`` (the sigmoid is taken where the gate is applied)."""
        return None if self.gate is None else self.gate(h, ctx)

    def write(self, y: torch.Tensor, gate: Optional[torch.Tensor], x: torch.Tensor, ctx: StepContext) -> None:
        pending = ctx.kernels.group_norm_step(x, groups=self.groups, eps=self.eps, y=y, gate=gate, post_weight=self.weight, mult=self.mult, defer=True)
        if ctx.may_defer:
            ctx.pending = pending
        else:
            ctx.kernels.finish(pending)


@BLOCKS.register("gated_sandwich")
class GatedSandwichBlock(Block):
    """The mixer behind ``norm1``, entering the stream through ``connect1``; then (if the layer has one) the feed-forward behind
    ``norm2`` through ``connect2``."""

    roles = ("norm1", "mixer", "connect1")
    defers_residual = True  # the stream is read through the norms only

    def __init__(self, parts: Dict[str, Part]):
        super().__init__(parts)
        unknown = [r for r in parts if r not in ("norm1", "mixer", "connect1", "norm2", "feed_forward", "connect2")]
        if unknown:
            raise ValueError(f"block 'gated_sandwich' has no role {', '.join(unknown)}")
        self.norm1, self.mixer, self.connect1 = parts["norm1"], parts["mixer"], parts["connect1"]
        self.feed_forward: Optional[Part] = parts.get("feed_forward")
        self.norm2, self.connect2 = parts.get("norm2"), parts.get("connect2")
        if self.feed_forward is not None and (self.norm2 is None or self.connect2 is None):
            raise ValueError("block 'gated_sandwich': a feed-forward needs norm2 and connect2")

    def _sublayer(self, norm, connect, run, x: torch.Tensor, ctx: StepContext) -> None:
        may_defer = ctx.may_defer
        if not norm.folds_pending:
            ctx.settle()
        h = norm(x, ctx)
        y = torch.empty_like(x)
        ctx.may_defer = False  # a sublayer's result is complete before it is gated and normed
        run(h, y)
        product = ctx.take_product_pending(y)
        if product is not None:
            ctx.kernels.finish(product)
        gate = connect.gate_of(h, ctx)
        ctx.may_defer = may_defer
        connect.write(y, gate, x, ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        self._sublayer(self.norm1, self.connect1, lambda h, y: self.mixer.compute(h, y, ctx, unit, writes_cache), x, ctx)
        if self.feed_forward is not None:
            self._sublayer(self.norm2, self.connect2, lambda h, y: self.feed_forward.compute(h, y, ctx), x, ctx)
