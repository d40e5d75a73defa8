"""A feed-forward made of many small experts of which every token uses a few (a mixture of experts).

With h the feed-forward's input and E experts: router logits z = W_router h (32-bit sums), scores s = sigmoid(z). The choice
goes by s + correction (a vector that only steers the choice); the experts form ``n_groups`` equal groups of neighbours, a
group's score is the sum of its ``group_top`` largest choice scores, and only experts of the ``keep`` best groups can be chosen
(the others count as minus infinity). The ``top`` experts with the largest choice scores run; the result is the sum of their
outputs weighted by their s (divided by the sum of the chosen s with ``renormalize``). An expert is
W_down (act(W_gate h) * (W_up h)) without biases.

Nothing of the routing goes to the host: a kernel orders the step's (token, choice) pairs by expert and cuts every expert's
stretch into row tiles, and the two products run over the tiles with a grid sized for the worst case (workgroups beyond the
tiles that exist return at once), so the launches depend on the number of tokens alone and a step can be replayed from a
HIP graph. Experts whose inner width is no multiple of 8 carry zeros behind it.

Switches beside that: ``score`` "softmax" (the scores are the softmax of z over all router outputs); ``n_identity`` router outputs
behind the experts' that stand for experts without weights whose result is their input (they take part in scores, groups and
choice like any other); ``limit`` and ``up_shift`` in the experts' activation, act(min(gate, limit)) * (clamp(up, +-limit) +
up_shift); ``shared``, the description of a feed-forward that runs for every token and is added.
"""
from __future__ import annotations

from typing import Dict

import torch

from levanter_amd.kernels.library import ACTIVATIONS
from .base import BuildEnv, FeedForward, StepContext
from .linear import Linear
from .embedding import tensors_of_nested
from .registry import FEED_FORWARDS, part_class
from .spec import PartSpec


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    """params: ``dim``, ``inner_dim``, ``n_experts``, ``top``, ``n_groups`` (1), ``keep`` (1), ``group_top`` (2), ``activation``
    ("silu"), ``renormalize`` (False), ``correction`` (True: the tensor exists), ``score`` ("sigmoid" or "softmax"), ``n_identity`` (0),
    ``limit`` (None), ``up_shift`` (0), ``shared`` (None, or the description of a feed-forward). Tensors: ``router.weight`` ``[E + n_identity, dim]``,
    ``correction`` ``[E + n_identity]``, and per expert e ``experts.<e>.gate.weight``, ``experts.<e>.up.weight`` ``[inner, dim]``,
    ``experts.<e>.down.weight`` ``[dim, inner]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim, self.inner, self.n_experts, self.top = int(p["dim"]), int(p["inner_dim"]), int(p["n_experts"]), int(p["top"])
        self.n_groups, self.keep, self.group_top = int(p.get("n_groups", 1)), int(p.get("keep", 1)), int(p.get("group_top", 2))
        self.activation = p.get("activation", "silu")
        self.renormalize = bool(p.get("renormalize", False))
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"routed_experts: unknown activation {self.activation!r}")
        E, D, F = self.n_experts, self.dim, self.inner
        self.n_identity = int(p.get("n_identity", 0))
        N = self.n_outputs = E + self.n_identity  # what the router chooses among
        self.score = p.get("score", "sigmoid")
        if self.score not in ("sigmoid", "softmax"):
            raise ValueError(f"routed_experts: the scores are 'sigmoid' or 'softmax', got {self.score!r}")
        self.limit = float(p["limit"]) if p.get("limit") else 0.0
        self.up_shift = float(p.get("up_shift", 0.0))
        if N % self.n_groups or not 0 < self.keep <= self.n_groups or not 0 < self.top <= self.keep * (N // self.n_groups):
            raise ValueError(f"routed_experts: {N} experts in {self.n_groups} groups, {self.keep} kept, {self.top} used")
        Fp = self.inner_padded = (F + 7) // 8 * 8

        def f32(name, shape):
            t = tensors[name].to(torch.float32).cpu()
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"routed_experts: {name} must be {list(shape)}, got {list(t.shape)}")
            return t

        self.router = Linear(f32("router.weight", (N, D)), None, "out_in", env)
        self.correction = f32("correction", (N,)).to(env.device).contiguous() if p.get("correction", True) else None
        shared: PartSpec = p.get("shared")
        self.shared = None
        if shared is not None:
            self.shared = part_class(shared.kind, shared.family or "feed_forward")(shared, tensors_of_nested("shared", tensors), env)
            self.graph_safe = bool(self.shared.graph_safe)
        # [E, gate rows then up rows, dim] and [E, dim, inner]
        w_in = torch.zeros(E, 2 * Fp, D)
        w_down = torch.zeros(E, D, Fp)
        for e in range(E):
            w_in[e, :F] = f32(f"experts.{e}.gate.weight", (F, D))
            w_in[e, Fp:Fp + F] = f32(f"experts.{e}.up.weight", (F, D))
            w_down[e, :, :F] = f32(f"experts.{e}.down.weight", (D, F))
        self.w_in = w_in.to(env.device, env.dtype).contiguous()
        self.w_down = w_down.to(env.device, env.dtype).contiguous()

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        self._run(h, x, ctx, True)

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext) -> None:
        self._run(h, y, ctx, False)

    def run_routed(self, h: torch.Tensor, z: torch.Tensor, y: torch.Tensor, ctx: StepContext) -> None:
        """The feed-forward's result into ``y`` from router logits ``z`` (float32 ``[T, E]``, rows may be strided) that a block has
        computed as part of a larger product over ``h``."""
        self._run(h, y, ctx, False, z)

    def _run(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext, accumulate: bool, z=None) -> None:
        K = ctx.kernels
        T, E, top = h.shape[0], self.n_outputs, self.top
        dev = h.device
        if z is None:
            z = self.router(h, ctx, out_dtype=torch.float32)
        if accumulate:
            ctx.settle()  # the sum below reads the residual stream itself
        chosen = torch.empty((T, top), dtype=torch.int32, device=dev)
        weights = torch.empty((T, top), dtype=torch.float32, device=dev)
        more = {"softmax": True} if self.score == "softmax" else {}
        K.moe_route(z, self.correction, chosen, weights, n_groups=self.n_groups, keep=self.keep, group_top=self.group_top, renormalize=self.renormalize, **more)
        P = T * top
        rows = K.moe_tile_rows(P, E)  # prompts: four row tiles on every weight fragment a wave loads
        tables = torch.empty(2 * P + 3 * K.moe_max_tiles(P, E, rows) + 1, dtype=torch.int32, device=dev)
        sorted_pairs, pos_of, meta, tiles = tables[:P], tables[P:2 * P], tables[2 * P:2 * P + 1], tables[2 * P + 1:]
        own = {"n_real": self.n_experts} if self.n_identity else {}
        K.moe_sort(chosen, E, sorted_pairs, pos_of, tiles, meta, tile_rows=rows, **own)
        inner = ctx.empty(P, self.inner_padded)
        clamp = {"limit": self.limit, "up_shift": self.up_shift} if self.limit or self.up_shift else {}
        K.moe_linear(h, self.w_in, inner, tiles, meta, sorted_pairs, top=top, gather=True, glu=True, activation=self.activation, tile_rows=rows, **clamp)
        expert_out = ctx.empty(P, self.dim, torch.float32)
        K.moe_linear(inner, self.w_down, expert_out, tiles, meta, sorted_pairs, top=top, gather=False, tile_rows=rows)
        if self.n_identity:
            K.moe_combine(expert_out, pos_of, weights, y, accumulate=accumulate, chosen=chosen, n_real=self.n_experts, identity_in=h)
        else:
            K.moe_combine(expert_out, pos_of, weights, y, accumulate=accumulate)
        if self.shared is not None:
            may_defer, ctx.may_defer = ctx.may_defer, False  # y is not the residual stream: its sum is finished here
            self.shared.forward(h, y, ctx)  # added to the experts' sum
            ctx.may_defer = may_defer
