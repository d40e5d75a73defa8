"""Embeddings: from token ids to the residual stream's first value. GPT-2: the token's row plus the row of its
absolute position (src/levanter/models/gpt2.py:291-308), summed in 32-bit by one kernel."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from levanter_amd.cache.requirements import SlotState
from .base import BuildEnv, Embedding, StepContext
from .registry import EMBEDDINGS, part_class
from .spec import PartSpec


def nested_tensors(spec: PartSpec, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The loaded tensors of a part under its local names. The tensors of a part nested in its parameters (an
    embedding's position encoding, an attention's rotation) travel along as ``<parameter>.<local name>``."""
    out = {local: tensors[ts.name] for local, ts in spec.tensors.items()}
    for param, v in spec.params.items():
        if isinstance(v, PartSpec):
            out.update({f"{param}.{k}": t for k, t in nested_tensors(v, tensors).items()})
    return out


def tensors_of_nested(param: str, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """What ``nested_tensors`` carried along for the part in parameter ``param``, under that part's local names."""
    prefix = param + "."
    return {k[len(prefix):]: t for k, t in tensors.items() if k.startswith(prefix)}


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Embedding):
    """params: ``vocab_size``, ``dim``, ``position`` (the description of a position encoding, or None), ``scale`` (a
    multiplier of the embedding's output, 1 by default), ``norm`` (the description of a norm that the residual stream's first
    value goes through, or None; its class takes ``out_dtype`` and gives float32), ``pairs`` (None, or ``{"buckets", "mul_prev",
    "mul_cur"}``: the row ``(token before * mul_prev + token * mul_cur) mod buckets`` of ``pairs.table`` ``[buckets + 1, dim]`` is added, the
    table's last row for a request's first token; the token before a step's first token is kept in the request's state slot); tensor
    ``table``."""

    STATE_UNIT = -1
    """The cache unit of the embedding's own per-request state (the plan's entries count from 0)."""

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.vocab_size = int(spec.params["vocab_size"])
        self.dim = int(spec.params["dim"])
        self.scale = float(spec.params.get("scale", 1.0))
        self.table = tensors["table"].to(env.device, env.dtype).contiguous()
        pos_spec: Optional[PartSpec] = spec.params.get("position")
        self.position = None
        if pos_spec is not None:
            self.position = part_class(pos_spec.kind, pos_spec.family or "position")(pos_spec, tensors_of_nested("position", tensors), env)
        self.pairs = spec.params.get("pairs")
        self.pair_table = None
        if self.pairs is not None:
            self.pair_table = tensors["pairs.table"].to(env.device, env.dtype).contiguous()
            if tuple(self.pair_table.shape) != (int(self.pairs["buckets"]) + 1, self.dim):
                raise ValueError(f"token_embedding: the pair table must be [{int(self.pairs['buckets']) + 1}, {self.dim}], got {list(self.pair_table.shape)}")
        norm_spec: Optional[PartSpec] = spec.params.get("norm")
        self.norm = None
        if norm_spec is not None:
            self.norm = part_class(norm_spec.kind, norm_spec.family or "norm")(norm_spec, tensors_of_nested("norm", tensors), env)

    @property
    def graph_safe(self) -> bool:
        return (self.position is None or bool(self.position.graph_safe)) and (self.norm is None or bool(self.norm.graph_safe))

    @property
    def max_positions(self) -> Optional[int]:
        return None if self.position is None else self.position.max_positions

    def cache_requirement(self):
        """What the embedding keeps per request between steps (None: nothing): the last token, for the pairs."""
        return None if self.pairs is None else SlotState((1,), "int32")

    def __call__(self, ctx: StepContext) -> torch.Tensor:
        x = ctx.empty(ctx.n_tokens, self.dim, torch.float32)
        pos_table = None if self.position is None else self.position.embedding_table()
        if self.scale == 1.0:
            ctx.kernels.embed(ctx.tokens, ctx.attention.positions, self.table, pos_table, x)
        else:
            ctx.kernels.embed(ctx.tokens, ctx.attention.positions, self.table, pos_table, x, scale=self.scale)
        if self.pairs is not None:
            last = ctx.units[self.STATE_UNIT].state.view(-1)
            ctx.kernels.pair_embed_add(ctx.tokens, ctx.attention.positions, ctx.token_slots, last, self.pair_table, x,
                                       int(self.pairs["buckets"]), int(self.pairs["mul_prev"]), int(self.pairs["mul_cur"]))
        if self.norm is not None:
            x = self.norm(x, ctx, out_dtype=torch.float32)
        return x
