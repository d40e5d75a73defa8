"""A recurrent mixer with a matrix state per head: a generalized delta rule.

With h the mixer's input, H heads of d channels: r = W_r h, k = W_k h, v = W_v h; a decay per head and key channel,
w = exp(-sharpness * sigmoid(W_w2 tanh(W_w1 h) + w0)) (a low-rank map, so w lies in (exp(-sharpness), 1)); a removal rate per
head and key channel, a = sigmoid(W_a h + b_a). With the unit key u = k / sqrt(sum(k^2) + key_eps) the state goes

    S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,        o_t = S_t^T r_t,

from S = 0: the state forgets channel by channel, takes out what it holds along the current key, and writes the new pair.
Each head's o is divided by its root mean square, the heads are multiplied by a weight and by sigmoid(W_g h), and go through
W_o.

What a request carries from step to step is the state alone, float32 ``[H, d, d]`` in its state slot. Everything from the
sigmoids to the head norm is 32-bit; the projections run in the compute dtype with 32-bit sums, the decay's second product
gives float32.
"""
from __future__ import annotations

from typing import Dict

import torch

from levanter_amd.cache.requirements import SlotState
from .base import BuildEnv, CacheUnitView, Mixer, StepContext
from .linear import Linear
from .registry import MIXERS
from .spec import PartSpec


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


@MIXERS.register("general_delta_rule")
class GeneralDeltaRule(Mixer):
    """params: ``dim``, ``n_heads``, ``head_dim``, ``decay_rank`` (optional: the tensors give it), ``sharpness``, ``key_eps``, ``norm_eps``. Tensors (``[out, in]``):
    ``r.weight``, ``k.weight``, ``v.weight``, ``gate.weight``, ``removal.weight`` ``[H*d, dim]``, ``removal.bias`` ``[H*d]``,
    ``decay_down.weight`` ``[rank, dim]``, ``decay_up.weight`` ``[H*d, rank]``, ``decay_up.bias`` ``[H*d]``, ``norm.weight`` ``[H*d]``,
    ``out.weight`` ``[dim, H*d]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim, self.n_heads, self.head_dim = int(p["dim"]), int(p["n_heads"]), int(p["head_dim"])
        self.rank = int(tensors["decay_down.weight"].shape[0])  # the tensor says it; the description may too
        if p.get("decay_rank") not in (None, -1, self.rank):
            raise ValueError(f"general_delta_rule: decay_down.weight has {self.rank} rows, the description says {p['decay_rank']}")
        self.sharpness, self.key_eps, self.norm_eps = float(p["sharpness"]), float(p["key_eps"]), float(p["norm_eps"])
        C = self.channels = self.n_heads * self.head_dim
        if self.head_dim > 256:
            raise ValueError(f"general_delta_rule: heads of {self.head_dim} channels (at most 256)")

        def f32(name, shape):
            t = tensors[name].to(torch.float32).cpu()
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"general_delta_rule: {name} must be {list(shape)}, got {list(t.shape)}")
            return t

        # one product for everything that reads h and needs no activation: [r | k | v | removal | gate], each part starting at a
        # multiple of 8 columns; the decay's low-rank map is two small products of its own (tanh between them)
        self.part = Cp = _pad8(C)
        fill = torch.zeros(Cp - C, self.dim)
        zb = torch.zeros(Cp)
        rp = self.rank_padded = _pad8(self.rank)
        weights = [torch.cat([f32(f"{n}.weight", (C, self.dim)), fill], 0) for n in ("r", "k", "v", "removal", "gate")]
        bias = torch.cat([zb, zb, zb, torch.cat([f32("removal.bias", (C,)), torch.zeros(Cp - C)]), zb])
        self.proj = Linear(torch.cat(weights, 0), bias, "out_in", env)
        self.decay_down = Linear(torch.cat([f32("decay_down.weight", (self.rank, self.dim)), torch.zeros(rp - self.rank, self.dim)], 0), None, "out_in", env)
        self.decay_up = Linear(torch.cat([f32("decay_up.weight", (C, self.rank)), torch.zeros(C, rp - self.rank)], 1), f32("decay_up.bias", (C,)), "out_in", env)
        self.norm_weight = f32("norm.weight", (C,)).to(env.device).contiguous()
        self.out = Linear(f32("out.weight", (self.dim, C)), tensors.get("out.bias"), "out_in", env)

    def cache_requirement(self):
        return SlotState((self.n_heads, self.head_dim, self.head_dim), "float32")

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.channels)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a, h)
        self.out(a, ctx, residual=x, final=True)

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.channels)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a, h)
        self.out(a, ctx, out=y, may_leave=True)

    def attend(self, p: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool, a: torch.Tensor, h: torch.Tensor = None) -> None:
        """Everything between the two products: ``p`` ``[T, r | k | v | removal | gate (| columns of others)]`` is what ``proj`` gives,
        ``h`` the mixer's input (for the decay's own products), ``a`` ``[T, H*d]`` takes what ``out`` reads. The request's state is
        read and advanced."""
        if not writes_cache:
            raise ValueError("general_delta_rule: a recurrence cannot read another entry's state without advancing it")
        K = ctx.kernels
        C, Cp = self.channels, self.part
        r, k, v, rem, g = (p[:, i * Cp:i * Cp + C] for i in range(5))
        w_pre = self.decay_up(self.decay_down(h, ctx, activation="tanh"), ctx, out_dtype=torch.float32)
        # a step with prompt portions has fewer runs than tokens (at most one per request of the step): the path for prompts
        max_runs = int(ctx.seq_slots.numel()) if ctx.attention.n_prefill_tiles else None
        K.delta_rule(r, k, v, rem, g, w_pre, self.norm_weight, unit.state, ctx.token_slots, a, self.n_heads, self.head_dim, self.norm_eps,
                     self.key_eps, self.sharpness, max_runs=max_runs)
