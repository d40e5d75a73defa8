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
    """params: ``dim``, ``groups``, ``eps``, ``weight_offset`` (0; 1 for a weight that is stored as its distance from one); tensor
    ``weight`` ``[dim]``. Folds a pending gated write of the same grouping into its pass."""

    graph_safe = True
    folds_pending = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.dim, self.groups, self.eps = int(spec.params["dim"]), int(spec.params["groups"]), float(spec.params["eps"])
        if self.dim % self.groups:
            raise ValueError(f"group_rmsnorm: {self.dim} numbers do not split into {self.groups} equal groups")
        self.weight = (tensors["weight"].to(env.device, torch.float32) + float(spec.params.get("weight_offset", 0.0))).contiguous()
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
    params: ``dim``, ``groups``, ``eps``, ``mult``, ``gate`` (False: no gate and no gate tensors), ``weight_offset`` (0; 1 for a weight
    that is stored as its distance from one). Tensors: ``weight`` ``[dim]``,
    ``gate.weight`` ``[dim, dim]``, ``gate.bias`` ``[dim]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim, self.groups, self.eps, self.mult = int(p["dim"]), int(p["groups"]), float(p["eps"]), float(p.get("mult", 1.0))
        self.weight = (tensors["weight"].to(env.device, torch.float32) + float(p.get("weight_offset", 0.0))).contiguous()
        self.gate = Linear(tensors["gate.weight"], tensors.get("gate.bias"), "out_in", env) if p.get("gate", True) else None
        if self.weight.numel() != self.dim or (self.gate is not None and (self.gate.n_in, self.gate.n_out) != (self.dim, self.dim)):
            raise ValueError("gated_post_norm: weights do not have the sizes of the description")

    def gate_of(self, h: torch.Tensor, ctx: StepContext) -> Optional[torch.Tensor]:
        """``gate.weight h + gate.bias`` (the sigmoid is taken where the gate is applied)."""
        return None if self.gate is None else self.gate(h, ctx)

    def fuse_behind(self, first: Linear, env: BuildEnv) -> Optional[Linear]:
        """One product for ``first`` and the gate, which read the same input: ``[first's rows | zeros up to a multiple of 8 | gate]``.
        The connection drops its own matrix; whoever runs the product hands the gate's columns (from ``gate_offset``) to ``write``.
        None if there is no gate or the two do not fit together."""
        if self.gate is None or first.weight.dtype != self.gate.weight.dtype or first.n_in != self.dim:
            return None
        dev = first.weight.device
        fill = (-first.n_out) % 8
        self.gate_offset = first.n_out + fill
        zeros = torch.zeros(fill, self.dim, dtype=first.weight.dtype, device=dev)
        b1 = first.bias if first.bias is not None else torch.zeros(first.n_out, device=dev)
        b2 = self.gate.bias if self.gate.bias is not None else torch.zeros(self.dim, device=dev)
        fused = Linear(torch.cat([first.weight, zeros, self.gate.weight], 0), torch.cat([b1, torch.zeros(fill, device=dev), b2]), "out_in", env)
        self.gate = None
        return fused

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
        # a sublayer's gate reads the sublayer's own input: where the sublayer offers its first product (a mixer's ``proj`` with
        # ``attend`` and ``out``, a feed-forward's ``router`` with ``run_routed``), the gate's rows join it and the parts drop theirs
        self.fused_mixer = self.fused_ff = None
        m, f = self.mixer, self.feed_forward
        if all(hasattr(m, a) for a in ("proj", "attend", "out")) and hasattr(self.connect1, "fuse_behind"):
            self.mixer_cols = m.proj.n_out
            self.fused_mixer = self.connect1.fuse_behind(m.proj, m.env)
            if self.fused_mixer is not None:
                m.proj = None
        if f is not None and all(hasattr(f, a) for a in ("router", "run_routed")) and hasattr(self.connect2, "fuse_behind"):
            self.router_cols = f.router.n_out
            self.fused_ff = self.connect2.fuse_behind(f.router, f.env)
            if self.fused_ff is not None:
                f.router = None

    def _sublayer(self, norm, connect, run, x: torch.Tensor, ctx: StepContext) -> None:
        """``run(h, y)`` computes the sublayer's result into ``y`` and gives the gate's sums if its first product has made them."""
        may_defer = ctx.may_defer
        if not norm.folds_pending:
            ctx.settle()
        h = norm(x, ctx)
        y = torch.empty_like(x)
        ctx.may_defer = False  # a sublayer's result is complete before it is gated and normed
        gate = run(h, y)
        product = ctx.take_product_pending(y)
        if product is not None:
            ctx.kernels.finish(product)
        if gate is None:
            gate = connect.gate_of(h, ctx)
        ctx.may_defer = may_defer
        connect.write(y, gate, x, ctx)

    def _run_mixer(self, h, y, ctx, unit, writes_cache):
        if self.fused_mixer is None:
            self.mixer.compute(h, y, ctx, unit, writes_cache)
            return None
        m = self.mixer
        pz = self.fused_mixer(h, ctx)  # [T, the mixer's projections | the gate]
        a = ctx.empty(h.shape[0], m.out.n_in)
        m.attend(pz[:, :self.mixer_cols], ctx, unit, writes_cache, a, h=h)
        m.out(a, ctx, out=y)
        return pz[:, self.connect1.gate_offset:self.connect1.gate_offset + self.connect1.dim]

    def _run_feed_forward(self, h, y, ctx):
        if self.fused_ff is None:
            self.feed_forward.compute(h, y, ctx)
            return None
        pz = self.fused_ff(h, ctx, out_dtype=torch.float32)  # the router's logits are 32-bit sums, so the gate's are too
        self.feed_forward.run_routed(h, pz[:, :self.router_cols], y, ctx)
        return pz[:, self.connect2.gate_offset:self.connect2.gate_offset + self.connect2.dim]

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        self._sublayer(self.norm1, self.connect1, lambda h, y: self._run_mixer(h, y, ctx, unit, writes_cache), x, ctx)
        if self.feed_forward is not None:
            self._sublayer(self.norm2, self.connect2, lambda h, y: self._run_feed_forward(h, y, ctx), x, ctx)


@BLOCKS.register("post_norm")
class PostNormBlock(Block):
    """Sublayers that read the residual stream itself and whose results are normed on their way into it:
    ``x <- x + connect1(mixer(x))``, then (if the layer has one) ``x <- x + connect2(feed_forward(x))``; a ``connect`` is a
    ``gated_post_norm`` (its gate may be switched off). There is no norm ahead of a sublayer: its input is the stream, rounded to
    the compute dtype by the pass that also does the write of the sublayer before (one row kernel a sublayer)."""

    roles = ("mixer", "connect1")
    defers_residual = True  # the stream is read through that pass only

    def __init__(self, parts: Dict[str, Part]):
        super().__init__(parts)
        unknown = [r for r in parts if r not in ("mixer", "connect1", "feed_forward", "connect2")]
        if unknown:
            raise ValueError(f"block 'post_norm' has no role {', '.join(unknown)}")
        self.mixer, self.connect1 = parts["mixer"], parts["connect1"]
        self.feed_forward: Optional[Part] = parts.get("feed_forward")
        self.connect2 = parts.get("connect2")
        if self.feed_forward is not None and self.connect2 is None:
            raise ValueError("block 'post_norm': a feed-forward needs connect2")

    @staticmethod
    def _read(connect, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        """The stream as a sublayer's input; the write that the sublayer before has left pending is done in the same pass."""
        pending = ctx.take_pending(x)
        if pending is not None and not (isinstance(pending, PendingGatedNorm) and pending.groups == connect.groups and pending.eps == connect.eps):
            ctx.kernels.finish(pending)
            pending = None
        h = ctx.empty(x.shape[0], x.shape[1])
        ctx.kernels.group_norm_step(x, groups=connect.groups, eps=connect.eps, h_out=h, pending=pending, plain_read=True)
        return h

    def _sublayer(self, connect, run, x: torch.Tensor, ctx: StepContext) -> None:
        may_defer = ctx.may_defer
        h = self._read(connect, x, ctx)
        y = torch.empty_like(x)
        ctx.may_defer = False  # a sublayer's result is complete before it is normed
        run(h, y)
        product = ctx.take_product_pending(y)
        if product is not None:
            ctx.kernels.finish(product)
        gate = connect.gate_of(h, ctx)
        ctx.may_defer = may_defer
        connect.write(y, gate, x, ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        self._sublayer(self.connect1, lambda h, y: self.mixer.compute(h, y, ctx, unit, writes_cache), x, ctx)
        if self.feed_forward is not None:
            self._sublayer(self.connect2, lambda h, y: self.feed_forward.compute(h, y, ctx), x, ctx)
