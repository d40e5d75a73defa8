"""A recurrent mixer with a matrix state per head that forgets by key channel: gated linear attention.

With h the mixer's input, H heads of dk key and dv value channels: q = W_q h, k = W_k h, v = W_v h; a decay per head and key
channel from a low-rank map, a = sigmoid(W_a2 (W_a1 h) + b_a2)^(1 / tau), so a lies in (0, 1) and tau sets how slowly the state
forgets. The state goes

    S_t = diag(a_t) S_(t-1) + k_t v_t^T,        o_t = S_t^T (q_scale q_t),

from S = 0. Each head's o is divided by its root mean square over dv and multiplied by a weight (one vector of dv for all heads,
or one per head), the heads are multiplied by gate(W_g h) (silu or sigmoid) and go through W_o.

What a request carries from step to step is the state alone, float32 ``[H, dk, dv]`` in its state slot. Everything from the
decay's sum to the head norm is 32-bit; the projections run in the compute dtype with 32-bit sums, the decay's second product
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


@MIXERS.register("gated_linear_attention")
class GatedLinearAttention(Mixer):
    """params: ``dim``, ``n_heads``, ``key_dim``, ``value_dim``, ``tau``, ``q_scale`` (``key_dim^(-1/2)`` by default), ``norm_eps``,
    ``gate`` ("silu" or "sigmoid"), ``decay_rank`` (optional: the tensors give it), ``out_scale`` (1: a branch's weight in a sum of
    branches). Tensors (``[out, in]``): ``q.weight``, ``k.weight`` ``[H*dk, dim]``, ``v.weight``, ``gate.weight`` ``[H*dv, dim]``,
    ``decay_down.weight`` ``[rank, dim]``, ``decay_up.weight`` ``[H*dk, rank]``, ``decay_up.bias`` ``[H*dk]``, ``norm.weight`` ``[dv]`` or
    ``[H*dv]``, ``out.weight`` ``[dim, H*dv]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim, self.n_heads, self.key_dim, self.value_dim = int(p["dim"]), int(p["n_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.tau, self.norm_eps = float(p["tau"]), float(p["norm_eps"])
        self.q_scale = float(p["q_scale"]) if p.get("q_scale") is not None else self.key_dim ** -0.5
        self.gate = p.get("gate", "silu")
        self.out_scale = float(p.get("out_scale", 1.0))
        if self.gate not in ("silu", "sigmoid"):
            raise ValueError(f"gated_linear_attention: the gate must be 'silu' or 'sigmoid', got {self.gate!r}")
        if self.tau <= 0 or max(self.key_dim, self.value_dim) > 256:
            raise ValueError(f"gated_linear_attention: tau={self.tau} must be positive and heads of {self.key_dim} / {self.value_dim} channels at most 256 wide")
        self.rank = int(tensors["decay_down.weight"].shape[0])  # the tensor says it; the description may too
        if p.get("decay_rank") not in (None, -1, self.rank):
            raise ValueError(f"gated_linear_attention: decay_down.weight has {self.rank} rows, the description says {p['decay_rank']}")
        H, dk, dv, D = self.n_heads, self.key_dim, self.value_dim, self.dim
        self.qk_cols, self.vg_cols = H * dk, H * dv

        def f32(name, shape):
            t = tensors[name].to(torch.float32).cpu()
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"gated_linear_attention: {name} must be {list(shape)}, got {list(t.shape)}")
            return t

        # one product for everything that reads h: [q | k | v | gate | the decay's inner sums], each part starting at a multiple of 8
        # columns; the decay's second product (from its inner sums to a 32-bit sum per key channel) is a small product of its own
        self.qk_part, self.vg_part = _pad8(self.qk_cols), _pad8(self.vg_cols)
        rows = []
        for name, n, padded in (("q", self.qk_cols, self.qk_part), ("k", self.qk_cols, self.qk_part), ("v", self.vg_cols, self.vg_part),
                                ("gate", self.vg_cols, self.vg_part)):
            rows += [f32(f"{name}.weight", (n, D)), torch.zeros(padded - n, D)]
        rp = self.rank_padded = _pad8(self.rank)
        rows += [f32("decay_down.weight", (self.rank, D)), torch.zeros(rp - self.rank, D)]
        self.proj = Linear(torch.cat(rows, 0), None, "out_in", env)
        self.decay_up = Linear(torch.cat([f32("decay_up.weight", (self.qk_cols, self.rank)), torch.zeros(self.qk_cols, rp - self.rank)], 1),
                               f32("decay_up.bias", (self.qk_cols,)), "out_in", env)
        nw = tensors["norm.weight"].to(torch.float32).cpu().reshape(-1)
        if nw.numel() == dv:
            nw = nw.repeat(H)  # one weight for all heads
        if nw.numel() != self.vg_cols:
            raise ValueError(f"gated_linear_attention: norm.weight must have {dv} or {self.vg_cols} entries, got {nw.numel()}")
        self.norm_weight = (nw * self.out_scale).to(env.device).contiguous()
        self.out = Linear(f32("out.weight", (D, self.vg_cols)), tensors.get("out.bias"), "out_in", env)

    def cache_requirement(self):
        return SlotState((self.n_heads, self.key_dim, self.value_dim), "float32")

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.vg_cols)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a)
        self.out(a, ctx, residual=x, final=True)

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.vg_cols)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a)
        self.out(a, ctx, out=y, may_leave=True)

    def attend(self, p: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool, a: torch.Tensor) -> None:
        """Everything between the two products: ``p`` ``[T, q | k | v | gate | decay's inner sums (| columns of others)]`` is what ``proj``
        gives, ``a`` ``[T, H*dv]`` takes what ``out`` reads. The request's state is read and advanced."""
        if not writes_cache:
            raise ValueError("gated_linear_attention: a recurrence cannot read another entry's state without advancing it")
        o1, o2, o3, o4 = self.qk_part, 2 * self.qk_part, 2 * self.qk_part + self.vg_part, 2 * self.qk_part + 2 * self.vg_part
        q, k = p[:, :self.qk_cols], p[:, o1:o1 + self.qk_cols]
        v, g = p[:, o2:o2 + self.vg_cols], p[:, o3:o3 + self.vg_cols]
        z = self.decay_up(p[:, o4:o4 + self.rank_padded], ctx, out_dtype=torch.float32)
        # a step with prompt portions has fewer runs than tokens (at most one per request of the step): the path for prompts
        max_runs = int(ctx.seq_slots.numel()) if ctx.attention.n_prefill_tiles else None
        ctx.kernels.gated_linear_attention(q, k, v, g, z, self.norm_weight, unit.state, ctx.token_slots, a, self.n_heads, self.key_dim, self.value_dim,
                                           self.tau, self.q_scale, self.norm_eps, gate=self.gate, max_runs=max_runs)
