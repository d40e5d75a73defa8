"""KegetarConfig: the configuration of the Kegetar architecture under its config.json keys.

config.json: ``architecture`` ("Kegetar"), ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` (the factor of every sublayer's
contribution), ``embedding.bigram`` (``buckets``, ``mul_prev``, ``mul_cur``: an embedding of the pair (token before, token) that is
added to the token's; absent: none) and ``layers``, a list with one entry per layer: ``type`` (the mixer: "parallel" or
"attention"), ``mixer`` (its sizes and constants), ``mlp`` (``kind`` "dense" with ``ff``; ``kind`` "moe" with ``expert`` (``ff``,
``limit``), ``router`` (``experts``, ``top``, optional ``identity`` and ``groups`` with ``count`` and ``keep``) and optional ``shared``
(``ff``, ``limit``); or null for a layer without a feed-forward) and optionally ``weights_of``: the index of an earlier layer whose
tensors this layer runs (that layer's own, or those it runs itself), with a cache and state of its own; its sizes must fit those
tensors. Layers may differ in all of it.

* parallel: ``left`` (an attention: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot`` with ``dims``, ``base`` and optional
  ``scaling`` (``factor``, ``original``, ``fast``, ``slow``), ``mask`` with ``size`` and ``keep_first``) and ``right`` (a linear attention:
  ``heads``, ``dim``, ``vdim``, ``tau``; optional ``decay_rank``, the inner size of the decay's low-rank map: a checkpoint's tensors give
  it, so only a model with drawn weights needs the key).
* attention: ``heads``, ``kv_heads``, ``dim`` (``vdim`` equals it: the keys are the values), ``scale``, ``mask.size``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, Tuple

from .lm_config import ConfigError, LmConfig

MIXER_TYPES = ("parallel", "attention")
MLP_KINDS = ("dense", "moe")


def _positive_int(v) -> bool:
    return isinstance(v, int) and not isinstance(v, bool) and v > 0


def _number(v) -> bool:
    return isinstance(v, (int, float)) and not isinstance(v, bool)


def _need_ints(where: str, d: dict, keys) -> None:
    for key in keys:
        if not _positive_int(d.get(key)):
            raise ConfigError(f"kegetar: {where}.{key} must be a positive integer, got {d.get(key)!r}")


def _check_mask(where: str, m: dict, keep_allowed: bool) -> None:
    mask = m.get("mask")
    if mask is None:
        return
    if not isinstance(mask, dict) or not (mask.get("size") is None or _positive_int(mask.get("size"))):
        raise ConfigError(f"kegetar: {where}.mask.size must be a positive integer, got {mask!r}")
    keep = mask.get("keep_first", 0)
    if not (isinstance(keep, int) and not isinstance(keep, bool) and keep >= 0) or (keep and not keep_allowed):
        raise ConfigError(f"kegetar: {where}.mask.keep_first must be a non-negative integer (and only this kind of attention has it), got {keep!r}")


def _check_softmax_attention(where: str, m: dict, keys_are_values: bool) -> None:
    m.setdefault("kv_heads", m.get("heads"))
    m.setdefault("vdim", m.get("dim"))
    _need_ints(where, m, ("heads", "kv_heads", "dim", "vdim"))
    if m["heads"] % m["kv_heads"]:
        raise ConfigError(f"kegetar: {where}: {m['heads']} heads are no multiple of {m['kv_heads']} key/value heads")
    if keys_are_values and m["vdim"] != m["dim"]:
        raise ConfigError(f"kegetar: {where}: the keys are the values, so vdim={m['vdim']} must equal dim={m['dim']}")
    if not _number(m.get("scale")):
        raise ConfigError(f"kegetar: {where}.scale must be a number, got {m.get('scale')!r}")
    _check_mask(where, m, keep_allowed=not keys_are_values)
    rot = m.get("rot")
    if rot is not None:
        if keys_are_values:
            raise ConfigError(f"kegetar: {where}: this attention has no rotation")
        if not isinstance(rot, dict) or not isinstance(rot.get("dims"), int) or rot["dims"] < 0 or rot["dims"] % 2 or rot["dims"] > m["dim"]:
            raise ConfigError(f"kegetar: {where}.rot.dims must be an even number of at most dim={m['dim']}, got {rot!r}")
        if not (_number(rot.get("base")) and rot["base"] > 1):
            raise ConfigError(f"kegetar: {where}.rot.base must be a number above 1, got {rot.get('base')!r}")
        sc = rot.get("scaling")
        if sc is not None:
            if not isinstance(sc, dict) or not all(_number(sc.get(k)) and sc[k] > 0 for k in ("factor", "original", "fast", "slow")):
                raise ConfigError(f"kegetar: {where}.rot.scaling needs positive factor, original, fast and slow, got {sc!r}")


def _check_mlp(where: str, mlp) -> None:
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
        raise ConfigError(f"kegetar: {where}: mlp.kind must be one of {', '.join(MLP_KINDS)}, got {mlp!r}")
    if mlp["kind"] == "dense":
        _need_ints(f"{where}: mlp", mlp, ("ff",))
        return
    expert, router = mlp.get("expert"), mlp.get("router")
    if not isinstance(expert, dict) or not _positive_int(expert.get("ff")) or not (_number(expert.get("limit")) and expert["limit"] > 0):
        raise ConfigError(f"kegetar: {where}: mlp.expert needs a positive integer ff and a positive limit, got {expert!r}")
    if not isinstance(router, dict):
        raise ConfigError(f"kegetar: {where}: mlp.router is missing")
    _need_ints(f"{where}: mlp.router", router, ("experts", "top"))
    ident = router.get("identity", 0)
    if not (isinstance(ident, int) and not isinstance(ident, bool) and ident >= 0):
        raise ConfigError(f"kegetar: {where}: mlp.router.identity must be a non-negative integer, got {ident!r}")
    groups = router.get("groups")
    if groups is None:
        groups = {"count": 1, "keep": 1}
    if not isinstance(groups, dict):
        raise ConfigError(f"kegetar: {where}: mlp.router.groups must be an object, got {groups!r}")
    _need_ints(f"{where}: mlp.router.groups", groups, ("count", "keep"))
    N, G, keep, top = router["experts"] + ident, groups["count"], groups["keep"], router["top"]
    if N % G or keep > G or top > keep * (N // G):
        raise ConfigError(f"kegetar: {where}: {N} router outputs in {G} groups, {keep} kept, {top} used do not fit together")
    shared = mlp.get("shared")
    if shared is not None and (not isinstance(shared, dict) or not _positive_int(shared.get("ff")) or not (_number(shared.get("limit")) and shared["limit"] > 0)):
        raise ConfigError(f"kegetar: {where}: mlp.shared needs a positive integer ff and a positive limit, got {shared!r}")


@LmConfig.register_subclass("kegetar")
@dataclass(frozen=True)
class KegetarConfig(LmConfig):
    vocab: int = 0
    width: int = 0
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    bigram: Any = None
    layers: Tuple[Dict[str, Any], ...] = ()
    initializer_range: float = 0.02

    def __post_init__(self):
        if not _positive_int(self.vocab) or not _positive_int(self.width):
            raise ConfigError(f"kegetar: vocab and width must be positive integers, got {self.vocab!r} and {self.width!r}")
        if not (_number(self.norm_eps) and self.norm_eps > 0):
            raise ConfigError(f"kegetar: norm.eps must be positive, got {self.norm_eps!r}")
        if not _number(self.residual_mult):
            raise ConfigError(f"kegetar: residual_mult must be a number, got {self.residual_mult!r}")
        if self.bigram is not None:
            if not isinstance(self.bigram, dict):
                raise ConfigError(f"kegetar: embedding.bigram must be an object, got {self.bigram!r}")
            _need_ints("embedding.bigram", self.bigram, ("buckets",))
            for key in ("mul_prev", "mul_cur"):
                v = self.bigram.get(key)
                if not (isinstance(v, int) and not isinstance(v, bool) and v >= 0):
                    raise ConfigError(f"kegetar: embedding.bigram.{key} must be a non-negative integer, got {v!r}")
        if not self.layers:
            raise ConfigError("kegetar: the configuration lists no layers")
        for i, layer in enumerate(self.layers):
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"kegetar: layer {i} has type {layer.get('type') if isinstance(layer, dict) else layer!r}; known: {', '.join(MIXER_TYPES)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"kegetar: layer {i} has no 'mixer' sizes")
            where = f"layer {i}: mixer"
            if layer["type"] == "parallel":
                left, right = m.get("left"), m.get("right")
                if not isinstance(left, dict) or not isinstance(right, dict):
                    raise ConfigError(f"kegetar: {where} needs 'left' and 'right'")
                _check_softmax_attention(f"{where}.left", left, keys_are_values=False)
                right.setdefault("vdim", right.get("dim"))
                _need_ints(f"{where}.right", right, ("heads", "dim", "vdim"))
                if not (_number(right.get("tau")) and right["tau"] > 0):
                    raise ConfigError(f"kegetar: {where}.right.tau must be positive, got {right.get('tau')!r}")
                if right.get("decay_rank") is not None and not _positive_int(right["decay_rank"]):
                    raise ConfigError(f"kegetar: {where}.right.decay_rank must be a positive integer, got {right['decay_rank']!r}")
            else:
                _check_softmax_attention(where, m, keys_are_values=True)
            _check_mlp(f"layer {i}", layer.get("mlp"))
            src = layer.get("weights_of")
            if src is not None:
                if not (isinstance(src, int) and not isinstance(src, bool) and 0 <= src < i):
                    raise ConfigError(f"kegetar: layer {i}: weights_of must name an earlier layer, got {src!r}")
                other = self.layers[self.owner_of(src)]
                if other.get("type") != layer["type"] or (other.get("mlp") or {}).get("kind") != (layer.get("mlp") or {}).get("kind"):
                    raise ConfigError(f"kegetar: layer {i} runs the weights of layer {self.owner_of(src)}, which is of another kind")

    def owner_of(self, i: int) -> int:
        """The layer whose tensors layer ``i`` runs: itself, or what its ``weights_of`` leads to."""
        while self.layers[i].get("weights_of") is not None:
            i = self.layers[i]["weights_of"]
        return i

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_hf_config(cls, hf_config: Dict[str, Any]) -> "KegetarConfig":
        for required in ("vocab", "width", "layers"):
            if required not in hf_config:
                raise ConfigError(f"kegetar: config.json lacks the key {required!r}")
        norm = hf_config.get("norm") or {}
        if not isinstance(norm, dict) or "eps" not in norm:
            raise ConfigError("kegetar: config.json lacks norm.eps")
        layers = hf_config["layers"]
        if not isinstance(layers, (list, tuple)):
            raise ConfigError("kegetar: 'layers' must be a list")
        emb = hf_config.get("embedding") or {}
        if not isinstance(emb, dict):
            raise ConfigError("kegetar: 'embedding' must be an object")
        extra = {"initializer_range": hf_config["initializer_range"]} if "initializer_range" in hf_config else {}
        return cls(vocab=hf_config["vocab"], width=hf_config["width"], norm_eps=norm["eps"], residual_mult=hf_config.get("residual_mult", 1.0),
                   bigram=copy.deepcopy(emb.get("bigram")), layers=tuple(copy.deepcopy(list(layers))), **extra)

    def to_hf_config(self) -> Dict[str, Any]:
        out = {"architecture": "Kegetar", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "residual_mult": self.residual_mult, "layers": copy.deepcopy(list(self.layers)), "initializer_range": self.initializer_range}
        if self.bigram is not None:
            out["embedding"] = {"bigram": copy.deepcopy(self.bigram)}
        return out

    def __hash__(self):
        return hash((self.vocab, self.width, self.norm_eps, self.residual_mult, repr(self.bigram), repr(self.layers)))

    def model_spec(self):
        from levanter_amd.models.kegetar import kegetar_model_spec

        return kegetar_model_spec(self)
