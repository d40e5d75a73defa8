"""Causal attention whose keys and values are both made from one small latent per token, which is all the cache keeps.

With h the mixer's input: q = W_q h (H heads of dk), c = RMSNorm(W_dkv h) (the latent, R numbers, with a weight), and per head
k_h = W_uk[h] c, v_h = W_uv[h] c. A score is q_h . k_h = q_h . (W_uk[h] c) = (W_uk[h]^T q_h) . c, and a head's output is
W_uv[h] (sum_j p_j c_j): so the pages hold c alone, as one key/value head of size R that all H query heads share, queries go
through W_uk[h]^T before attention and the attention's result through W_uv[h] after it. Both are block-diagonal products
(one block per head); a decoding step reads R numbers per cached token instead of H (dk + dv).

The page layouts of keys and values differ (each is what the matrix instructions read), so a latent is stored in both; the
attention kernel is the one for heads with separate key and value sizes, with one key/value head. Latents whose size is no
multiple of what the kernels take are stored with zeros behind them (rows of zeros in W_dkv and the matching columns of
W_uk, W_uv), which changes neither a score nor an output; the norm divides by the true size.

Switched on by the description:

* queries through a latent of their own: q = W_uq RMSNorm(W_dq h) (``query_latent_dim``);
* a rotated part: every query head carries ``rope_dim`` more dimensions behind its dk, and W_dkv h ``rope_dim`` more rows behind
  the latent (not normed): one key part that all heads share. Both turn with the position (``rotary``: ``dims`` <= rope_dim
  dimensions in the rotate-half layout, dimension i paired with i + dims/2, angle p * base^(-2i/dims)), and the score is
  scale * (q_h . k_h + q_rot_h . k_rot). The cached key is [c | k_rot] (after the rotation), the cached value c: the queries'
  rotated part passes the map into the latent's space unchanged (an identity block);
* a window of the last ``window`` keys;
* a sink per head: exp(sink_h) in the softmax's denominator, with no key and no value (``sinks``);
* an output gate: head h times sigmoid(gate_h . h) (``gate``);
* a layer without W_dkv that reads the latent and rotated key part another layer has cached (``shared_kv``): its plan entry
  names that layer's cache unit and does not write. ``cache_window`` is what the unit keeps: the largest window of the
  layers that read it.
"""
from __future__ import annotations

from typing import Dict

import torch

from levanter_amd.cache.requirements import PagedKv
from .base import BuildEnv, CacheUnitView, Mixer, StepContext
from .linear import Linear
from .registry import MIXERS
from .spec import PartSpec


def _pad(n: int, step: int) -> int:
    return (n + step - 1) // step * step


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    """params: ``dim``, ``n_heads``, ``head_dim``, ``value_dim``, ``latent_dim``, ``scale``, ``norm_eps``; optional ``query_latent_dim``,
    ``rope_dim`` with ``rotary`` (``{"dims", "base"}``), ``window``, ``cache_window``, ``sinks``, ``gate``, ``shared_kv``. Tensors
    (``[out, in]``): ``q.weight`` ``[H*(dk+dr), dim]`` or, with a query latent, ``q_down.weight`` ``[Q, dim]``, ``q_norm.weight``
    ``[Q]``, ``q.weight`` ``[H*(dk+dr), Q]``; ``down.weight`` ``[R+dr, dim]``, ``latent_norm.weight`` ``[R]`` (not with ``shared_kv``);
    ``up_k.weight`` ``[H*dk, R]``, ``up_v.weight`` ``[H*dv, R]``, ``out.weight`` ``[dim, H*dv]``; ``sinks`` ``[H]``; ``gate.weight`` ``[H, dim]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim, self.n_heads = int(p["dim"]), int(p["n_heads"])
        self.head_dim, self.value_dim, self.true_latent = int(p["head_dim"]), int(p["value_dim"]), int(p["latent_dim"])
        self.scale, self.eps = float(p["scale"]), float(p["norm_eps"])
        self.true_rope = int(p.get("rope_dim") or 0)
        self.true_q_latent = int(p.get("query_latent_dim") or 0)
        self.window = p.get("window")
        self.cache_window = p.get("cache_window", self.window)
        self.shared_kv = bool(p.get("shared_kv", False))
        H, dk, dv, R, dr, Q = self.n_heads, self.head_dim, self.value_dim, self.true_latent, self.true_rope, self.true_q_latent
        # the cache keeps keys in chunks of 8 elements, the matrix-core kernels work on tiles of 16
        step = 16 if env.dtype == torch.bfloat16 else 8
        self.latent = Rp = _pad(R, step)
        self.rope = drp = _pad(dr, step)
        self.q_latent = Qp = _pad(Q, 8)
        self.key_dim = Rp + drp
        self.q_head = dk + dr

        def f32(name, shape):
            t = tensors[name].to(torch.float32).cpu()
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"latent_attention: {name} must be {list(shape)}, got {list(t.shape)}")
            return t

        rot = p.get("rotary") or {}
        n_pairs = int(rot.get("dims", 0)) // 2
        if 2 * n_pairs > dr:
            raise ValueError(f"latent_attention: {2 * n_pairs} rotated dimensions do not fit a rotated part of {dr}")
        self.freqs = None
        if n_pairs:
            base = float(rot["base"])
            self.freqs = torch.tensor([base ** (-2.0 * i / (2 * n_pairs)) for i in range(n_pairs)], dtype=torch.float64).to(torch.float32).to(env.device)
        # one product for everything that reads h: [queries or their latent | latent | rotated key part | gate], each part
        # starting at a multiple of 8 columns
        rows, at = [], 0

        def part(w, width):
            nonlocal at
            start = at
            rows.extend([w, torch.zeros(width - w.shape[0], self.dim)])
            at += width
            return start

        self.q_norm_weight = self.up_q = None
        if Q:
            self.q_cols = Qp
            part(f32("q_down.weight", (Q, self.dim)), Qp)
            self.q_norm_weight = torch.cat([f32("q_norm.weight", (Q,)), torch.zeros(Qp - Q)]).to(env.device).contiguous()
            self.up_q = Linear(torch.cat([f32("q.weight", (H * self.q_head, Q)), torch.zeros(H * self.q_head, Qp - Q)], 1), None, "out_in", env)
        else:
            self.q_cols = H * self.q_head
            part(f32("q.weight", (H * self.q_head, self.dim)), _pad(self.q_cols, 8))
        self.c_off = at
        self.norm_weight = None
        if not self.shared_kv:
            w_down = f32("down.weight", (R + dr, self.dim))
            part(w_down[:R], Rp)
            if drp:
                part(w_down[R:], drp)
            self.norm_weight = torch.cat([f32("latent_norm.weight", (R,)), torch.zeros(Rp - R)]).to(env.device).contiguous()
        self.g_off = at
        self.has_gate = bool(p.get("gate", False))
        if self.has_gate:
            part(f32("gate.weight", (H, self.dim)), _pad(H, 8))
        self.proj = Linear(torch.cat(rows, 0), None, "out_in", env)
        self.sinks = f32("sinks", (H,)).to(env.device).contiguous() if p.get("sinks") else None
        # queries into the latent's space, head by head: [H, Rp + drp, dk + dr] = [[W_uk[h]^T, 0], [0, 1]]; results out of it:
        # [H, dv, Rp] = W_uv[h]
        w_uk, w_uv = f32("up_k.weight", (H * dk, R)), f32("up_v.weight", (H * dv, R))
        absorb = torch.zeros(H, self.key_dim, self.q_head)
        absorb[:, :R, :dk] = w_uk.view(H, dk, R).transpose(1, 2)
        for i in range(dr):
            absorb[:, Rp + i, dk + i] = 1.0
        self.w_absorb = absorb.contiguous().to(env.device, env.dtype)
        self.w_expand = torch.cat([w_uv.view(H, dv, R), torch.zeros(H, dv, Rp - R)], 2).contiguous().to(env.device, env.dtype)
        self.out = Linear(f32("out.weight", (self.dim, H * dv)), tensors.get("out.bias"), "out_in", env)

    def cache_requirement(self):
        return PagedKv(1, self.key_dim, self.cache_window, value_dim=self.latent if self.rope else None)

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.n_heads * self.value_dim)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a)
        self.out(a, ctx, residual=x, final=True)

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.n_heads * self.value_dim)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a)
        self.out(a, ctx, out=y, may_leave=True)

    def attend(self, p: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool, a: torch.Tensor, h=None) -> None:
        """Everything between the two products: ``p`` ``[T, q | latent (| columns of others)]`` is what ``proj`` gives, ``a``
        ``[T, heads * value_dim]`` (rows may be strided) takes the heads that ``out`` reads. (``h``, the mixer's input, is not needed.)"""
        K = ctx.kernels
        T, H, Rp, KD = p.shape[0], self.n_heads, self.latent, self.key_dim
        g = unit.group
        if writes_cache == self.shared_kv:
            raise ValueError("latent_attention: a layer with a latent of its own writes its cache unit, one that shares another's only reads")
        positions = ctx.attention.positions
        if self.up_q is not None:  # the queries' latent: RMS norm (32-bit statistics, the weight applied), in place; then the heads
            K.head_prepare(p, 1, self.q_latent, self.eps, norm_dim=self.true_q_latent, norm_weight=self.q_norm_weight)
            q = self.up_q(p[:, :self.q_latent], ctx)
        else:
            q = p[:, :self.q_cols]
        singles = ctx.attention.n_prefill_tiles == 0  # a step of single tokens: rotation, norm and cache write in one kernel
        if self.freqs is not None and not (singles and writes_cache and self.rope):
            K.rotary_half(q, H, self.q_head, self.head_dim, self.freqs, positions)
        if writes_cache:
            kv = p[:, self.c_off:self.c_off + KD]  # [latent | rotated key part]
            c = kv[:, :Rp]
            if singles and self.rope:
                K.latent_rope_write(kv, Rp, self.norm_weight, self.eps, self.true_latent, q, H, self.q_head, self.head_dim, self.freqs, positions,
                                    unit.k_pages, unit.v_pages, g.dest, g.page_size)
            elif singles:
                K.norm_write_latent(c, self.norm_weight, self.eps, self.true_latent, unit.k_pages, unit.v_pages, g.dest, g.page_size)
            else:
                if self.freqs is not None:
                    K.rotary_half(kv, 1, KD, Rp, self.freqs, positions)
                # the latent's RMS norm (32-bit statistics, the weight applied), in place; then into the pages, as key and as value
                K.head_prepare(c, 1, Rp, self.eps, norm_dim=self.true_latent, norm_weight=self.norm_weight)
                K.kv_write(kv, c, unit.k_pages, unit.v_pages, g.dest, 1, KD, g.page_size, value_dim=Rp)  # 16 tokens at a time, transposed through LDS
        qa = ctx.empty(T, H * KD)
        K.block_linear(q, self.w_absorb, None, qa)
        o = torch.empty((T, H, 1, Rp), dtype=torch.float32, device=p.device)
        extra = {} if self.sinks is None else {"sinks": self.sinks}
        K.attention_values(qa, o, unit.k_pages, unit.v_pages, ctx.attention, n_heads=H, n_kv_heads=1, head_dim=KD, value_dim=Rp,
                           all_value_heads=False, page_size=g.page_size, scale=self.scale, window=self.window, block_tables=g.block_tables, **extra)
        if self.has_gate:  # head h times sigmoid(gate_h): a number per head commutes with the map out of the latent's space
            og = ctx.empty(T, H * Rp)
            K.head_talk(o, None, p[:, self.g_off:self.g_off + H], og, H, 1, Rp)
            K.block_linear(og, self.w_expand, None, a)
        else:
            K.block_linear(o.view(T, H * Rp), self.w_expand, None, a)  # takes the 32-bit result as it is
