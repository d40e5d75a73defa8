"""TativikConfig: the configuration of the Tativik architecture under its config.json keys.

config.json: ``architecture`` ("Tativik"), ``vocab``, ``width``, ``norm`` (``eps`` and ``groups``: every norm of the residual
stream splits the vector into that many equal parts), ``residual_mult`` (the factor of every sublayer's contribution) and
``layers``, a list with one entry per layer: ``type`` (the mixer: "latent_attention" or "general_delta"), ``mixer`` (its sizes
and constants) and ``mlp`` (``kind`` "moe" with ``expert.ff`` and ``router``: ``experts``, ``top``, optional ``groups`` with
``count`` and ``keep``; or null for a layer without a feed-forward). Layers may differ in all of it.

* latent_attention: ``heads``, ``dim`` unrotated and ``rot_dim`` rotated dimensions of a query/key head, ``vdim`` of a value head,
  ``kv_rank`` the size of the cached latent, ``q_rank`` the size of the queries' latent, ``scale``, ``rot`` (``dims``, ``base``),
  ``mask.size`` the window (absent: all keys), ``kv_from`` (absent, or the index of an earlier layer whose cached latent and
  rotated key part this layer reads instead of making its own).
* general_delta: ``heads``, ``dim`` channels a head; optional ``decay_rank`` (the inner size of the decay's low-rank map: a
  checkpoint's tensors give it, so only a model with drawn weights needs the key).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, Tuple

from .lm_config import ConfigError, LmConfig

MIXER_TYPES = ("latent_attention", "general_delta")
MLP_KINDS = ("moe",)


def _positive_int(v) -> bool:
    return isinstance(v, int) and not isinstance(v, bool) and v > 0


def _number(v) -> bool:
    return isinstance(v, (int, float)) and not isinstance(v, bool)


def _need_ints(where: str, d: dict, keys) -> None:
    for key in keys:
        if not _positive_int(d.get(key)):
            raise ConfigError(f"tativik: {where}.{key} must be a positive integer, got {d.get(key)!r}")


def _check_latent(where: str, m: dict, index: int, layers) -> None:
    m.setdefault("vdim", m.get("dim"))
    m.setdefault("rot_dim", 0)
    _need_ints(where, m, ("heads", "dim", "vdim", "kv_rank", "q_rank"))
    if not (isinstance(m["rot_dim"], int) and not isinstance(m["rot_dim"], bool) and m["rot_dim"] >= 0):
        raise ConfigError(f"tativik: {where}.rot_dim must be a non-negative integer, got {m['rot_dim']!r}")
    if not _number(m.get("scale")):
        raise ConfigError(f"tativik: {where}.scale must be a number, got {m.get('scale')!r}")
    mask = m.get("mask")
    if mask is not None and not (isinstance(mask, dict) and (mask.get("size") is None or _positive_int(mask.get("size")))):
        raise ConfigError(f"tativik: {where}.mask must be {{'size': positive integer}}, got {mask!r}")
    rot = m.get("rot")
    if rot is not None:
        if not isinstance(rot, dict) or not isinstance(rot.get("dims"), int) or rot["dims"] < 0 or rot["dims"] % 2 or rot["dims"] > m["rot_dim"]:
            raise ConfigError(f"tativik: {where}.rot.dims must be an even number of at most rot_dim={m['rot_dim']}, got {rot!r}")
        if not (_number(rot.get("base")) and rot["base"] > 0):
            raise ConfigError(f"tativik: {where}.rot.base must be a positive number, got {rot.get('base')!r}")
    src = m.get("kv_from")
    if src is not None:
        if not (isinstance(src, int) and not isinstance(src, bool) and 0 <= src < index):
            raise ConfigError(f"tativik: {where}.kv_from must name an earlier layer, got {src!r}")
        other = layers[src]
        om = other.get("mixer") if isinstance(other, dict) else None
        if other.get("type") != "latent_attention" or not isinstance(om, dict) or om.get("kv_from") is not None:
            raise ConfigError(f"tativik: {where}.kv_from = {src}: that layer has no latent of its own")
        same = ("kv_rank", "rot_dim")
        if any(om.get(k, 0) != m.get(k, 0) for k in same) or (om.get("rot") or None) != (m.get("rot") or None):
            raise ConfigError(f"tativik: {where}.kv_from = {src}: kv_rank, rot_dim and rot of the two layers differ")


@LmConfig.register_subclass("tativik")
@dataclass(frozen=True)
class TativikConfig(LmConfig):
    vocab: int = 0
    width: int = 0
    norm_eps: float = 1e-6
    norm_groups: int = 1
    residual_mult: float = 1.0
    layers: Tuple[Dict[str, Any], ...] = ()
    initializer_range: float = 0.02

    def __post_init__(self):
        if not _positive_int(self.vocab) or not _positive_int(self.width):
            raise ConfigError(f"tativik: vocab and width must be positive integers, got {self.vocab!r} and {self.width!r}")
        if not (_number(self.norm_eps) and self.norm_eps > 0):
            raise ConfigError(f"tativik: norm.eps must be positive, got {self.norm_eps!r}")
        if not _positive_int(self.norm_groups) or self.width % self.norm_groups:
            raise ConfigError(f"tativik: norm.groups must divide the width {self.width}, got {self.norm_groups!r}")
        if not _number(self.residual_mult):
            raise ConfigError(f"tativik: residual_mult must be a number, got {self.residual_mult!r}")
        if not self.layers:
            raise ConfigError("tativik: the configuration lists no layers")
        for i, layer in enumerate(self.layers):
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"tativik: layer {i} has type {layer.get('type') if isinstance(layer, dict) else layer!r}; known: {', '.join(MIXER_TYPES)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"tativik: layer {i} has no 'mixer' sizes")
            where = f"layer {i}: mixer"
            if layer["type"] == "latent_attention":
                _check_latent(where, m, i, self.layers)
            else:
                _need_ints(where, m, ("heads", "dim"))
                if m.get("decay_rank") is not None and not _positive_int(m["decay_rank"]):
                    raise ConfigError(f"tativik: {where}.decay_rank must be a positive integer, got {m['decay_rank']!r}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"tativik: layer {i}: mlp.kind must be one of {', '.join(MLP_KINDS)}, got {mlp!r}")
                expert, router = mlp.get("expert"), mlp.get("router")
                if not isinstance(expert, dict) or not _positive_int(expert.get("ff")):
                    raise ConfigError(f"tativik: layer {i}: mlp.expert.ff must be a positive integer, got {expert!r}")
                if not isinstance(router, dict):
                    raise ConfigError(f"tativik: layer {i}: mlp.router is missing")
                _need_ints(f"layer {i}: mlp.router", router, ("experts", "top"))
                groups = router.get("groups")
                if groups is None:
                    groups = {"count": 1, "keep": 1}
                if not isinstance(groups, dict):
                    raise ConfigError(f"tativik: layer {i}: mlp.router.groups must be an object, got {groups!r}")
                _need_ints(f"layer {i}: mlp.router.groups", groups, ("count", "keep"))
                E, G, keep, top = router["experts"], groups["count"], groups["keep"], router["top"]
                if E % G or keep > G or top > keep * (E // G):
                    raise ConfigError(f"tativik: layer {i}: {E} experts in {G} groups, {keep} kept, {top} used do not fit together")

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_hf_config(cls, hf_config: Dict[str, Any]) -> "TativikConfig":
        for required in ("vocab", "width", "layers"):
            if required not in hf_config:
                raise ConfigError(f"tativik: config.json lacks the key {required!r}")
        norm = hf_config.get("norm") or {}
        if not isinstance(norm, dict) or "eps" not in norm:
            raise ConfigError("tativik: config.json lacks norm.eps")
        layers = hf_config["layers"]
        if not isinstance(layers, (list, tuple)):
            raise ConfigError("tativik: 'layers' must be a list")
        extra = {"initializer_range": hf_config["initializer_range"]} if "initializer_range" in hf_config else {}
        return cls(vocab=hf_config["vocab"], width=hf_config["width"], norm_eps=norm["eps"], norm_groups=norm.get("groups", 1),
                   residual_mult=hf_config.get("residual_mult", 1.0), layers=tuple(copy.deepcopy(list(layers))), **extra)

    def to_hf_config(self) -> Dict[str, Any]:
        return {"architecture": "Tativik", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "residual_mult": self.residual_mult, "layers": copy.deepcopy(list(self.layers)), "initializer_range": self.initializer_range}

    def __hash__(self):
        return hash((self.vocab, self.width, self.norm_eps, self.norm_groups, self.residual_mult, repr(self.layers)))

    def model_spec(self):
        from levanter_amd.models.tativik import tativik_model_spec

        return tativik_model_spec(self)
