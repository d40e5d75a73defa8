"""Causal self-attention over the paged cache whose pieces are switched on by its description:

* separate projections for queries, keys, values (and a gate), held as one matrix so that they are one product;
* key and value heads of different sizes;
* queries and keys divided by their root mean square per head (no weight), or (``qk_norm``) an RMS norm with a weight, per head
  with one weight for all query heads and one for all key heads, or over the whole projection at once; it comes before the rotation;
* no value projection (``values_from_keys``): the keys as projected, before any norm, are the values;
* a soft cap on the scaled score, then a term per head that grows with the distance, ``- slope[h] * (i - j)``;
* a rotation of queries and keys by their positions before the keys are cached (``rotary``: a position encoding);
* a window of the last ``window`` keys whose first ``keep_first`` positions stay in sight whatever the window, and/or chunks: a query sees only the keys of its own ``chunk`` positions, counted
  from the start of the sequence;
* the softmax weights mixed over the heads after the softmax, ``w'_h = sum_g talk[h, g] w_g``, each head applying its
  mixed weights to the values of its own key/value head;
* values blended with the values that an earlier layer computed for the same token (``value_mix``: the layer that is the
  "source" leaves its values in ``ctx.shared``, a layer that says "blend" caches ``(1 - l) v + l v_source``);
* the output of head h multiplied by ``sigmoid(gate_h(x))`` (or, ``gate_kind`` "element", every element of the heads by the sigmoid
  of a projection of its own) before the output projection, and all heads by ``out_scale``
  (the mixer's weight where a layer adds several mixers).

Scores, softmax, the unit norms, the blend and the mixing over heads are 32-bit in every precision. The mixing is done
after the weights have been applied: the attention kernel gives, for every query head, its weights applied to the values
of every key/value head, and a small kernel sums over the query heads (the two orders differ in rounding only).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from levanter_amd.cache.requirements import PagedKv
from .base import BuildEnv, CacheUnitView, Mixer, StepContext
from .embedding import tensors_of_nested
from .linear import Linear
from .registry import MIXERS, part_class
from .spec import PartSpec


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


@MIXERS.register("talking_heads_attention")
class TalkingHeadsAttention(Mixer):
    """params: ``dim``, ``n_heads``, ``n_kv_heads``, ``head_dim``, ``value_dim``, ``scale``, ``window`` (None: all keys),
    ``softcap`` (None: none), ``unit_norm_eps`` (None: queries and keys stay as projected), ``distance_slopes`` (one number
    per head, or None), ``value_mix`` (None, "source" or "blend") and ``value_mix_key`` (the name under which layers that
    belong together share values), ``chunk`` (None: none), ``rotary`` (the description of a position encoding with a
    ``rotate``, or None), ``out_scale`` (1 by default), ``qk_norm`` (None, "head" or "projection") with ``qk_norm_eps`` and the tensors
    ``q_norm.weight`` / ``k_norm.weight`` (``[head_dim]``, or the whole projection's size), ``keep_first`` (0), ``gate_kind`` ("head" or
    "element": ``gate.weight`` ``[heads * value_dim, dim]``), ``values_from_keys`` (False; True: no ``v.weight``). All tensors but the four matrices are optional. Tensors: ``q.weight``, ``k.weight``, ``v.weight``, ``out.weight`` (``[out, in]``), their
    optional ``.bias``, optional ``gate.weight`` ``[heads, dim]``, ``talk`` ``[heads, heads]``, ``value_mix.weight`` (one number)."""

    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim = int(p["dim"])
        self.n_heads, self.n_kv_heads = int(p["n_heads"]), int(p["n_kv_heads"])
        self.head_dim, self.value_dim = int(p["head_dim"]), int(p["value_dim"])
        self.scale = float(p["scale"])
        self.window: Optional[int] = p.get("window")
        self.chunk: Optional[int] = p.get("chunk")
        self.out_scale = float(p.get("out_scale", 1.0))
        self.softcap = p.get("softcap")
        self.unit_norm_eps = p.get("unit_norm_eps")
        self.keep_first = int(p.get("keep_first") or 0)
        self.qk_norm = p.get("qk_norm")
        if self.qk_norm not in (None, "head", "projection"):
            raise ValueError(f"attention: qk_norm must be None, 'head' or 'projection', got {self.qk_norm!r}")
        if self.qk_norm is not None and self.unit_norm_eps is not None:
            raise ValueError("attention: queries and keys are normed once: unit_norm_eps or qk_norm")
        self.qk_norm_eps = float(p.get("qk_norm_eps", 0.0))
        self.gate_elements = p.get("gate_kind", "head") == "element"
        self.values_from_keys = bool(p.get("values_from_keys", False))
        if self.values_from_keys and self.value_dim != self.head_dim:
            raise ValueError("attention: keys that are the values too need value_dim == head_dim")
        if self.n_heads % self.n_kv_heads != 0:
            raise ValueError(f"attention: {self.n_heads} heads are not a multiple of {self.n_kv_heads} key/value heads")
        # The cache keeps keys in chunks of 8 elements and the matrix-core kernels work on tiles of 16: heads of any other
        # size are stored with zeros behind them (rows of zeros in the projections, columns of zeros in the output
        # projection). Zeros change no score and no output; only the unit norm has to divide by the true size.
        step = 16 if env.dtype == torch.bfloat16 else 8
        self.true_head_dim, self.true_value_dim = self.head_dim, self.value_dim
        self.head_dim = (self.head_dim + step - 1) // step * step
        self.value_dim = (self.value_dim + step - 1) // step * step
        slopes = p.get("distance_slopes")
        self.slopes = None
        if slopes is not None:
            if len(slopes) != self.n_heads:
                raise ValueError(f"attention: {len(slopes)} slopes for {self.n_heads} heads")
            self.slopes = torch.tensor([float(s) for s in slopes], dtype=torch.float32, device=env.device)
        self.value_mix = p.get("value_mix")
        if self.value_mix not in (None, "source", "blend"):
            raise ValueError(f"attention: value_mix must be None, 'source' or 'blend', got {self.value_mix!r}")
        self.value_mix_key = "value_mix." + str(p.get("value_mix_key", "values"))
        self.blend = None
        if self.value_mix == "blend":
            self.blend = tensors["value_mix.weight"].to(env.device, torch.float32).reshape(1).contiguous()
        talk = tensors.get("talk")
        self.talk = None if talk is None else talk.to(env.device, torch.float32).contiguous()
        if self.talk is not None and tuple(self.talk.shape) != (self.n_heads, self.n_heads):
            raise ValueError(f"attention: the matrix that mixes the heads must be [{self.n_heads}, {self.n_heads}]")

        # one matrix for all projections of the mixer's input: queries, keys, values, gate; each starts at a multiple of 8 columns
        self.q_cols, self.k_cols, self.v_cols = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim, self.n_kv_heads * self.value_dim
        names = ["q", "k", "v"] + (["gate"] if "gate.weight" in tensors else [])
        sizes = {"q": self.q_cols, "k": self.k_cols, "v": self.v_cols, "gate": self.n_heads * self.value_dim if self.gate_elements else self.n_heads}
        # (heads, size in the checkpoint, size as stored here) of each projection
        heads_of = {"q": (self.n_heads, self.true_head_dim, self.head_dim), "k": (self.n_kv_heads, self.true_head_dim, self.head_dim),
                    "v": (self.n_kv_heads, self.true_value_dim, self.value_dim),
                    "gate": (self.n_heads, self.true_value_dim, self.value_dim) if self.gate_elements else (1, self.n_heads, self.n_heads)}
        rows, biases, self.offsets, at = [], [], {}, 0
        any_bias = any(f"{n}.bias" in tensors for n in names)
        self.q_norm_weight = self.k_norm_weight = None
        if self.qk_norm is not None:
            def norm_weight(name: str, nh: int) -> torch.Tensor:
                w = tensors[f"{name}.weight"].to(torch.float32).cpu().reshape(-1)
                per = 1 if self.qk_norm == "head" else nh  # heads that the weight spans
                if w.numel() != per * self.true_head_dim:
                    raise ValueError(f"attention: {name}.weight must have {per * self.true_head_dim} entries, got {w.numel()}")
                if self.head_dim != self.true_head_dim:  # zeros where the heads carry zeros
                    w = torch.cat([w.view(per, self.true_head_dim), torch.zeros(per, self.head_dim - self.true_head_dim)], 1).reshape(-1)
                return w.to(env.device).contiguous()

            self.q_norm_weight, self.k_norm_weight = norm_weight("q_norm", self.n_heads), norm_weight("k_norm", self.n_kv_heads)
        for n in names:
            nh, true, stored = heads_of[n]
            src = "k" if n == "v" and self.values_from_keys else n  # the value rows of the product are the key rows once more
            w = tensors[f"{src}.weight"].to(torch.float32).cpu()
            if tuple(w.shape) != (nh * true, self.dim):
                raise ValueError(f"attention: {n}.weight must be [{nh * true}, {self.dim}], got {list(w.shape)}")
            b = tensors.get(f"{src}.bias")
            b = torch.zeros(nh * true) if b is None else b.to(torch.float32).cpu()
            if stored != true:  # zeros behind every head
                w = torch.cat([w.view(nh, true, self.dim), torch.zeros(nh, stored - true, self.dim)], 1).reshape(nh * stored, self.dim)
                b = torch.cat([b.view(nh, true), torch.zeros(nh, stored - true)], 1).reshape(nh * stored)
            pad = _pad8(sizes[n]) - sizes[n]
            self.offsets[n] = at
            rows += [w, torch.zeros(pad, self.dim)]
            biases += [b, torch.zeros(pad)]
            at += sizes[n] + pad
        if self.offsets["k"] != self.q_cols:
            raise ValueError("attention: heads * head_dim must be a multiple of 8 (keys follow the queries without a gap)")
        self.proj = Linear(torch.cat(rows, 0), torch.cat(biases, 0) if any_bias else None, "out_in", env)
        self.has_gate = "gate" in self.offsets
        w_out = tensors["out.weight"]
        if p.get("weight_layout", "out_in") == "in_out":
            w_out = w_out.t()
        if tuple(w_out.shape) != (self.dim, self.n_heads * self.true_value_dim):
            raise ValueError("attention: the output projection does not have the sizes of the description")
        if self.value_dim != self.true_value_dim:  # columns of zeros where the heads carry zeros
            w_out = torch.cat([w_out.to(torch.float32).cpu().reshape(self.dim, self.n_heads, self.true_value_dim),
                               torch.zeros(self.dim, self.n_heads, self.value_dim - self.true_value_dim)], 2).reshape(self.dim, -1)
        self.out = Linear(w_out, tensors.get("out.bias"), "out_in", env)
        rotary = p.get("rotary")
        self.rotary = None
        if rotary is not None:  # it turns the heads as they are stored here: a head's zeros lie behind what it rotates
            rotary = PartSpec(rotary.kind, {**rotary.params, "head_dim": self.head_dim}, rotary.tensors, rotary.family)
            self.rotary = part_class(rotary.kind, rotary.family or "position")(rotary, tensors_of_nested("rotary", tensors), env)
            self.graph_safe = bool(self.rotary.graph_safe)

    def cache_requirement(self):
        return PagedKv(self.n_kv_heads, self.head_dim, self.window, None if self.value_dim == self.head_dim else self.value_dim, self.chunk,
                       **({"keep_first": self.keep_first} if self.keep_first else {}))

    def compute(self, h: torch.Tensor, y: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.n_heads * self.value_dim)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a)
        self.out(a, ctx, out=y, may_leave=True)

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        a = ctx.empty(h.shape[0], self.n_heads * self.value_dim)
        self.attend(self.proj(h, ctx), ctx, unit, writes_cache, a)
        self.out(a, ctx, residual=x, final=True)

    def attend(self, p: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool, a: torch.Tensor) -> None:
        """Everything between the two products: ``p`` ``[T, q | k | v | gate (| columns of others)]`` is what ``proj`` gives for
        the mixer's input, ``a`` ``[T, heads * value_dim]`` (rows may be strided) takes the gated heads that ``out`` reads. A
        block that runs ``proj`` and ``out`` as parts of larger products calls this directly."""
        K = ctx.kernels
        T = p.shape[0]
        o = self.offsets
        q = p[:, :self.q_cols]
        k = p[:, o["k"]:o["k"] + self.k_cols]
        v = p[:, o["v"]:o["v"] + self.v_cols]
        gate = p[:, o["gate"]:o["gate"] + (self.n_heads * self.value_dim if self.gate_elements else self.n_heads)] if self.has_gate else None
        single = writes_cache and ctx.attention.n_prefill_tiles == 0
        fused_rotation = {}
        fused_norm = {}
        if self.qk_norm == "projection":  # one statistic over all heads of a token: a pass of its own, ahead of everything else
            K.head_prepare(q, 1, self.q_cols, self.qk_norm_eps, norm_dim=self.n_heads * self.true_head_dim, norm_weight=self.q_norm_weight)
            K.head_prepare(k, 1, self.k_cols, self.qk_norm_eps, norm_dim=self.n_kv_heads * self.true_head_dim, norm_weight=self.k_norm_weight)
        elif self.qk_norm == "head":
            fused_norm = {"q_norm_weight": self.q_norm_weight, "k_norm_weight": self.k_norm_weight}
        rot_here = self.rotary is not None and getattr(self.rotary, "freqs", None) is not None and getattr(self.rotary, "head_dim", None) == self.head_dim
        if self.rotary is not None and rot_here and (single or fused_norm):
            # a step of single tokens: the rotation happens inside the kernel that writes the pages; with a weighted norm ahead of it,
            # a step with longer runs does both in one kernel of the same arithmetic (a norm with a weight does not commute with the rotation)
            fused_rotation = {"rotary_freqs": self.rotary.freqs, "positions": ctx.attention.positions} if self.rotary.freqs.numel() else {}
            if fused_rotation and getattr(self.rotary, "magnitude", 1.0) != 1.0:
                fused_rotation["rotary_magnitude"] = self.rotary.magnitude
        if fused_norm and (not single or (self.rotary is not None and not rot_here)):
            K.head_norm_rotate(q, k, self.n_heads, self.n_kv_heads, self.head_dim, self.qk_norm_eps, norm_dim=self.true_head_dim, **fused_norm, **fused_rotation)
            if self.rotary is not None and not rot_here:  # a rotation of another kind: behind the norm
                self.rotary.rotate(q, k, ctx)
            fused_norm, fused_rotation = {}, {}  # both are done: what writes the pages only writes
        elif self.rotary is not None and not (single and rot_here):
            self.rotary.rotate(q, k, ctx)
        v_first = None
        if self.value_mix == "source":
            ctx.shared[self.value_mix_key] = v
        elif self.value_mix == "blend":
            v_first = ctx.shared.get(self.value_mix_key)
            if v_first is None or v_first.shape != v.shape:
                raise RuntimeError("attention: no layer before this one has left values of this shape to blend with")
        g = unit.group
        if single:
            # a step of single tokens: unit norms, the rotation, the blend and the write into the pages are one kernel
            K.head_prepare_write(q, k, v, unit.k_pages, unit.v_pages, g.dest, self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim,
                                 g.page_size, self.qk_norm_eps if fused_norm else self.unit_norm_eps, v_first=v_first, blend=self.blend,
                                 norm_dim=self.true_head_dim, **fused_rotation, **fused_norm)
        else:
            n_norm = self.n_heads + self.n_kv_heads if self.unit_norm_eps is not None else 0
            if n_norm or v_first is not None:
                K.head_prepare(p[:, :self.q_cols + self.k_cols], n_norm, self.head_dim, self.unit_norm_eps or 0.0, v=v, v_first=v_first,
                               n_blend=self.n_kv_heads if v_first is not None else 0, value_dim=self.value_dim, blend=self.blend,
                               norm_dim=self.true_head_dim)
            if writes_cache:  # keys and values of 16 tokens at a time, transposed through LDS
                K.kv_write(k, v, unit.k_pages, unit.v_pages, g.dest, self.n_kv_heads, self.head_dim, g.page_size, value_dim=self.value_dim)
        nv = self.n_kv_heads if self.talk is not None else 1
        w = torch.empty((T, self.n_heads, nv, self.value_dim), dtype=torch.float32, device=p.device)
        K.attention_values(q, w, unit.k_pages, unit.v_pages, ctx.attention, n_heads=self.n_heads, n_kv_heads=self.n_kv_heads,
                           head_dim=self.head_dim, value_dim=self.value_dim, all_value_heads=self.talk is not None,
                           page_size=g.page_size, scale=self.scale, window=self.window, block_tables=g.block_tables,
                           softcap=self.softcap, slopes=self.slopes, **({"chunk": self.chunk} if self.chunk else {}),
                           **({"keep_first": self.keep_first} if self.keep_first else {}))
        K.head_talk(w, self.talk, gate, a, self.n_heads, self.n_kv_heads, self.value_dim, **({"out_scale": self.out_scale} if self.out_scale != 1.0 else {}),
                    **({"gate_elements": True} if self.gate_elements and gate is not None else {}))
