"""Kegetar as a model description: which parts each layer has and where their tensors come from.

The residual stream starts as the token's row of ``embed`` plus a row of ``bigram`` chosen by a hash of (token before, token). A
layer's sublayers read the stream itself and are normed on their way into it: x <- x + m N(mixer(x), 1 + norm1), then the same
with the feed-forward and ``norm2``; N is the RMS norm, m is ``residual_mult``. The mixer (``l<i>.mix.*``) is one of two:

* ``parallel``: half the sum of two branches, each through an RMS norm over the width with a weight of its own (``left.out``,
  ``right.out``). ``left``: softmax attention over a window that also keeps the request's first positions in sight, per-head RMS
  norm of queries and keys with one weight each (``q.norm``, ``k.norm``), rotation of neighbouring pairs with frequencies stretched
  along a ramp, an output gate per element (``g``), ``o``. ``right``: gated linear attention (``q``, ``k``, ``v``, the decay's low-rank
  map ``a1``, ``a2``, ``a2.b``, the head norm's weight ``norm``, the silu gate ``g``, ``o``).
* ``attention``: softmax attention without a value projection (the keys as projected are the values), queries and keys with
  biases and an RMS norm over the whole projection (``q.norm``, ``k.norm``), a distance term per head instead of a rotation, a
  plain window.

The feed-forward is dense (``gate``, ``up``, ``down`` with biases, tanh-gelu on the gate) or a mixture of experts
(``router``, ``correction``, ``e<j>.{gate,up,down}``, ``shared.{gate,up,down}``) with softmax scores, router outputs without experts
behind them that return their input, and a clamped activation. A layer with ``weights_of`` runs an earlier layer's tensors with a
cache unit of its own. ``final.norm`` (stored as its distance from one, as ``norm1`` and ``norm2``) comes before the head ``head``.
Linear weights are stored ``[out, in]``.
"""
from __future__ import annotations

import math

from levanter_amd.config.kegetar import KegetarConfig
from levanter_amd.parts.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry, TensorSpec

ROTATION_MAGNITUDE_SLOPE = 0.1  # cosine and sine are multiplied by ROTATION_MAGNITUDE_SLOPE * ln(factor) + 1 where frequencies are stretched
BRANCH_WEIGHT = 0.5  # the mixer 'parallel' is half the sum of its branches
GROUP_SCORE_TOP = 1  # a group of experts is scored by its largest choice score
EXPERT_UP_SHIFT = 1.0  # an expert multiplies its activated gate by (up + 1)
DISTANCE_SLOPE_RANGE = 8.0  # head h of H takes 2^(-DISTANCE_SLOPE_RANGE (h + 1) / H) a position off its scores


def kegetar_model_spec(cfg: KegetarConfig) -> ModelSpec:
    d, eps = cfg.width, float(cfg.norm_eps)
    lin = 1.0 / math.sqrt(d)

    def connection(name: str) -> PartSpec:
        return PartSpec("gated_post_norm", {"dim": d, "groups": 1, "eps": eps, "mult": float(cfg.residual_mult), "gate": False, "weight_offset": 1.0},
                        {"weight": TensorSpec(name, (d,), std=0.1)}, family="stream_mix")

    def left_attention(p: str, m: dict) -> PartSpec:
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        mask, rot = m.get("mask") or {}, m.get("rot")
        rotary = None
        if rot is not None and rot["dims"]:
            sc = rot.get("scaling")
            rotary = PartSpec("rotary_pairs", {"dims": rot["dims"], "base": float(rot["base"]), "scaling": dict(sc) if sc else None,
                                               "magnitude": ROTATION_MAGNITUDE_SLOPE * math.log(float(sc["factor"])) + 1.0 if sc else 1.0}, family="position")
        return PartSpec("talking_heads_attention",
                        {"dim": d, "n_heads": H, "n_kv_heads": G, "head_dim": dk, "value_dim": dv, "scale": float(m["scale"]), "window": mask.get("size"),
                         "keep_first": int(mask.get("keep_first", 0)) if mask.get("size") else 0, "qk_norm": "head", "qk_norm_eps": eps, "gate_kind": "element",
                         "rotary": rotary},
                        {"q.weight": TensorSpec(f"{p}.q", (H * dk, d), std=lin), "k.weight": TensorSpec(f"{p}.k", (G * dk, d), std=lin),
                         "v.weight": TensorSpec(f"{p}.v", (G * dv, d), std=lin), "q_norm.weight": TensorSpec(f"{p}.q.norm", (dk,), init="one_plus_normal", std=0.1),
                         "k_norm.weight": TensorSpec(f"{p}.k.norm", (dk,), init="one_plus_normal", std=0.1),
                         "gate.weight": TensorSpec(f"{p}.g", (H * dv, d), std=lin), "out.weight": TensorSpec(f"{p}.o", (d, H * dv), std=1.0 / math.sqrt(H * dv))},
                        family="mixer")

    def right_attention(p: str, m: dict) -> PartSpec:
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        rank = m.get("decay_rank") or -1
        return PartSpec("gated_linear_attention",
                        {"dim": d, "n_heads": H, "key_dim": dk, "value_dim": dv, "tau": float(m["tau"]), "q_scale": dk ** -0.5, "norm_eps": eps, "gate": "silu",
                         "decay_rank": rank},
                        {"q.weight": TensorSpec(f"{p}.q", (H * dk, d), std=lin), "k.weight": TensorSpec(f"{p}.k", (H * dk, d), std=lin),
                         "v.weight": TensorSpec(f"{p}.v", (H * dv, d), std=lin), "gate.weight": TensorSpec(f"{p}.g", (H * dv, d), std=lin),
                         "decay_down.weight": TensorSpec(f"{p}.a1", (rank, d), std=lin),
                         "decay_up.weight": TensorSpec(f"{p}.a2", (H * dk, rank), std=1.0 / math.sqrt(max(rank, 1))),
                         "decay_up.bias": TensorSpec(f"{p}.a2.b", (H * dk,), std=1.0),
                         "norm.weight": TensorSpec(f"{p}.norm", (dv,), init="one_plus_normal", std=0.1),
                         "out.weight": TensorSpec(f"{p}.o", (d, H * dv), std=1.0 / math.sqrt(H * dv))}, family="mixer")

    def parallel(p: str, m: dict) -> PartSpec:
        return PartSpec("parallel_mixers", {"left": left_attention(f"{p}.left", m["left"]), "right": right_attention(f"{p}.right", m["right"]),
                                            "left_scale": BRANCH_WEIGHT, "right_scale": BRANCH_WEIGHT, "branch_norm_eps": eps},
                        {"left_norm.weight": TensorSpec(f"{p}.left.out", (d,), init="one_plus_normal", std=0.1),
                         "right_norm.weight": TensorSpec(f"{p}.right.out", (d,), init="one_plus_normal", std=0.1)}, family="mixer")

    def keys_as_values_attention(p: str, m: dict) -> PartSpec:
        H, G, dk = m["heads"], m["kv_heads"], m["dim"]
        slopes = [2.0 ** (-DISTANCE_SLOPE_RANGE * (h + 1) / H) for h in range(H)]
        return PartSpec("talking_heads_attention",
                        {"dim": d, "n_heads": H, "n_kv_heads": G, "head_dim": dk, "value_dim": dk, "scale": float(m["scale"]),
                         "window": (m.get("mask") or {}).get("size"), "qk_norm": "projection", "qk_norm_eps": eps, "values_from_keys": True,
                         "distance_slopes": slopes},
                        {"q.weight": TensorSpec(f"{p}.q", (H * dk, d), std=lin), "q.bias": TensorSpec(f"{p}.q.b", (H * dk,), std=0.1),
                         "k.weight": TensorSpec(f"{p}.k", (G * dk, d), std=lin), "k.bias": TensorSpec(f"{p}.k.b", (G * dk,), std=0.1),
                         "q_norm.weight": TensorSpec(f"{p}.q.norm", (H * dk,), init="one_plus_normal", std=0.1),
                         "k_norm.weight": TensorSpec(f"{p}.k.norm", (G * dk,), init="one_plus_normal", std=0.1),
                         "out.weight": TensorSpec(f"{p}.o", (d, H * dk), std=1.0 / math.sqrt(H * dk))}, family="mixer")

    def gated(p: str, f: int, activation: str, biases: bool, limit=None, up_shift: float = 0.0) -> PartSpec:
        tensors = {"gate.weight": TensorSpec(f"{p}.gate", (f, d), std=lin), "up.weight": TensorSpec(f"{p}.up", (f, d), std=lin),
                   "down.weight": TensorSpec(f"{p}.down", (d, f), std=1.0 / math.sqrt(f))}
        if biases:
            tensors.update({"gate.bias": TensorSpec(f"{p}.gate.b", (f,), std=0.1), "up.bias": TensorSpec(f"{p}.up.b", (f,), std=0.1),
                            "down.bias": TensorSpec(f"{p}.down.b", (d,), std=0.1)})
        return PartSpec("gated_mlp", {"dim": d, "inner_dim": f, "activation": activation, "limit": limit, "up_shift": up_shift}, tensors, family="feed_forward")

    def experts(p: str, mlp: dict) -> PartSpec:
        f, limit, router = mlp["expert"]["ff"], float(mlp["expert"]["limit"]), mlp["router"]
        E, ident = router["experts"], int(router.get("identity", 0))
        g = router.get("groups") or {"count": 1, "keep": 1}
        tensors = {"router.weight": TensorSpec(f"{p}.router", (E + ident, d), std=lin), "correction": TensorSpec(f"{p}.correction", (E + ident,), std=0.02)}
        for e in range(E):
            tensors[f"experts.{e}.gate.weight"] = TensorSpec(f"{p}.e{e}.gate", (f, d), std=lin)
            tensors[f"experts.{e}.up.weight"] = TensorSpec(f"{p}.e{e}.up", (f, d), std=lin)
            tensors[f"experts.{e}.down.weight"] = TensorSpec(f"{p}.e{e}.down", (d, f), std=1.0 / math.sqrt(f))
        shared = mlp.get("shared")
        return PartSpec("routed_experts",
                        {"dim": d, "inner_dim": f, "n_experts": E, "n_identity": ident, "top": router["top"], "n_groups": g["count"], "keep": g["keep"],
                         "group_top": GROUP_SCORE_TOP, "score": "softmax", "activation": "quick_gelu", "limit": limit, "up_shift": EXPERT_UP_SHIFT,
                         "renormalize": False, "correction": True,
                         "shared": None if shared is None else gated(f"{p}.shared", shared["ff"], "quick_gelu", False, float(shared["limit"]), EXPERT_UP_SHIFT)},
                        tensors, family="feed_forward")

    def same(a: dict, b: dict) -> bool:
        return all(a.get(key) == b.get(key) for key in ("type", "mixer", "mlp"))

    layers, plan, layer_of = [], [], {}
    for i, layer in enumerate(cfg.layers):
        owner = cfg.owner_of(i)
        if owner != i and same(layer, cfg.layers[owner]):  # the earlier layer's built parts, a cache unit of its own
            layer_of[i] = layer_of[owner]
        else:  # tensors of its own, or the owner's tensors under constants of its own (another window, say): parts of its own
            p, m = f"l{owner}", layer["mixer"]
            mixer = parallel(f"{p}.mix", m) if layer["type"] == "parallel" else keys_as_values_attention(f"{p}.mix", m)
            parts = {"mixer": mixer, "connect1": connection(f"{p}.norm1")}
            mlp = layer.get("mlp")
            if mlp is not None:
                parts["feed_forward"] = gated(f"{p}.mlp", mlp["ff"], "gelu_new", True) if mlp["kind"] == "dense" else experts(f"{p}.mlp", mlp)
                parts["connect2"] = connection(f"{p}.norm2")
            layer_of[i] = len(layers)
            layers.append(LayerSpec("post_norm", parts))
        plan.append(PlanEntry(layer=layer_of[i], cache=i, writes_cache=True))

    emb_tensors = {"table": TensorSpec("embed", (cfg.vocab, d), std=1.0)}
    pairs = None
    if cfg.bigram is not None:
        pairs = {k: int(cfg.bigram[k]) for k in ("buckets", "mul_prev", "mul_cur")}
        emb_tensors["pairs.table"] = TensorSpec("bigram", (pairs["buckets"] + 1, d), std=0.5)
    embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "dim": d, "position": None, "pairs": pairs}, emb_tensors, family="embedding")
    head = PartSpec("linear_head", {"vocab_size": cfg.vocab, "dim": d}, {"weight": TensorSpec("head", (cfg.vocab, d), std=lin)}, family="head")
    final_norm = PartSpec("group_rmsnorm", {"dim": d, "groups": 1, "eps": eps, "weight_offset": 1.0}, {"weight": TensorSpec("final.norm", (d,), std=0.1)},
                          family="norm")
    return ModelSpec(
        architecture="kegetar",
        vocab_size=cfg.vocab,
        dim=d,
        embedding=embedding,
        layers=layers,
        plan=plan,
        final_norm=final_norm,
        head=head,
        max_positions=None,
        init_std=cfg.initializer_range,
    )
