"""Feed-forwards. Dense two-matrix unit: down(act(up(h))) (src/levanter/models/gpt2.py:150-155);
the activation runs in 32-bit inside the first product's epilogue, the residual sum in the second's."""
from __future__ import annotations

from typing import Dict

import torch

from levanter_amd.kernels.library import ACTIVATIONS
from .base import BuildEnv, FeedForward, StepContext
from .linear import Linear
from .registry import FEED_FORWARDS
from .spec import PartSpec


@FEED_FORWARDS.register("dense_mlp")
class DenseMlp(FeedForward):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.activation = p["activation"]
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"dense_mlp: unknown activation {self.activation!r}")
        layout = p.get("weight_layout", "out_in")
        self.up = Linear(tensors["up.weight"], tensors.get("up.bias"), layout, env)
        self.down = Linear(tensors["down.weight"], tensors.get("down.bias"), layout, env)
        if (self.up.n_in, self.up.n_out) != (p["dim"], p["inner_dim"]) or (self.down.n_in, self.down.n_out) != (p["inner_dim"], p["dim"]):
            raise ValueError("dense_mlp: weights do not have the sizes of the description")

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        m = self.up(h, ctx, activation=self.activation)
        self.down(m, ctx, residual=x, final=True)

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext) -> None:
        self.down(self.up(h, ctx, activation=self.activation), ctx, out=y, may_leave=True)


@FEED_FORWARDS.register("gated_mlp")
class GatedMlp(FeedForward):
    """down(act(gate h) * (up h + up_shift)): the two first products are one (gate rows, then up rows), the activation is a row
    kernel in 32-bit between the products. With ``limit`` the gate's sums are capped at it and the up sums clamped to +-limit
    before the activation. params: ``dim``, ``inner_dim``, ``activation``, ``limit`` (None), ``up_shift`` (0). Tensors ``[out, in]``:
    ``gate.weight``, ``up.weight`` ``[inner, dim]``, ``down.weight`` ``[dim, inner]``, optional ``.bias`` of each. An inner width that
    is no multiple of 8 carries zeros behind it."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.activation = p["activation"]
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"gated_mlp: unknown activation {self.activation!r}")
        D, F = int(p["dim"]), int(p["inner_dim"])
        self.limit = float(p["limit"]) if p.get("limit") else 0.0
        self.up_shift = float(p.get("up_shift", 0.0))
        Fp = self.inner_padded = (F + 7) // 8 * 8

        def f32(name, shape):
            t = tensors[name].to(torch.float32).cpu()
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"gated_mlp: {name} must be {list(shape)}, got {list(t.shape)}")
            return t

        w_in = torch.zeros(2 * Fp, D)
        w_in[:F], w_in[Fp:Fp + F] = f32("gate.weight", (F, D)), f32("up.weight", (F, D))
        b_in = None
        if "gate.bias" in tensors or "up.bias" in tensors:
            b_in = torch.zeros(2 * Fp)
            if "gate.bias" in tensors:
                b_in[:F] = f32("gate.bias", (F,))
            if "up.bias" in tensors:
                b_in[Fp:Fp + F] = f32("up.bias", (F,))
        self.up = Linear(w_in, b_in, "out_in", env)
        w_down = torch.zeros(D, Fp)
        w_down[:, :F] = f32("down.weight", (D, F))
        self.down = Linear(w_down, tensors.get("down.bias"), "out_in", env)

    def _inner(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        z = self.up(h, ctx)
        m = z[:, :self.inner_padded]
        ctx.kernels.glu_activate(z, m, self.activation, limit=self.limit, up_shift=self.up_shift)
        return m

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        self.down(self._inner(h, ctx), ctx, residual=x, final=True)

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext) -> None:
        self.down(self._inner(h, ctx), ctx, out=y, may_leave=True)


@FEED_FORWARDS.register("poly_norm_mlp")
class PolyNormMlp(FeedForward):
    """down(act(up(h))) with an activation that needs a token's whole row: c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, powers
    element by element, N(u) = u / sqrt(mean(u^2) + eps) over the inner width. The statistics and the sum are 32-bit and
    run as a kernel of their own between the two products. Tensors: ``up.weight``, ``down.weight`` (optional biases),
    ``coefficients`` [4]."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        layout = p.get("weight_layout", "out_in")
        self.eps = float(p["eps"])
        self.up = Linear(tensors["up.weight"], tensors.get("up.bias"), layout, env)
        self.down = Linear(tensors["down.weight"], tensors.get("down.bias"), layout, env)
        if (self.up.n_in, self.up.n_out) != (p["dim"], p["inner_dim"]) or (self.down.n_in, self.down.n_out) != (p["inner_dim"], p["dim"]):
            raise ValueError("poly_norm_mlp: weights do not have the sizes of the description")
        self.coefficients = tensors["coefficients"].to(env.device, torch.float32).contiguous()
        if self.coefficients.numel() != 4:
            raise ValueError(f"poly_norm_mlp: four coefficients, got {self.coefficients.numel()}")

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        z = self.up(h, ctx)
        self.activate(z, ctx, z)
        self.down(z, ctx, residual=x, final=True)

    def activate(self, z: torch.Tensor, ctx: StepContext, out: torch.Tensor) -> None:
        """What lies between the two products: ``z`` ``[T, inner_dim]`` -> ``out`` (may be ``z``; rows may be strided). A block
        that runs ``up`` and ``down`` as parts of larger products calls this directly."""
        ctx.kernels.poly_norm(z, self.coefficients, self.eps, out)
