"""Tativik as a model description: which parts each layer has and where their tensors come from.

The residual stream starts as the token's row of ``embed`` through the model's norm (``embed.norm``): an RMS norm in
``norm.groups`` groups, as every norm of the stream. A layer has a norm before and after each sublayer and a gate on the
sublayer's result: x <- x + m gn(mixer(gn(x, norm1)) * sigmoid(rg1 h + rg1.b), norm1b), then the same with the feed-forward,
``norm2``, ``rg2``, ``norm2b``; m is ``residual_mult``. The mixer (``l<i>.mix.*``) is one of two:

* ``latent_attention``: queries through a latent (``dq``, its RMS norm ``dq.norm``, ``uq``), keys and values from a cached latent
  (``dkv`` with ``dkv.norm``, ``uk``, ``uv``) plus one rotated key part that all heads share (the last ``rot_dim`` rows of ``dkv``),
  rotate-half rotary positions on the rotated parts, a sliding window, a sink per head in the softmax's denominator (``sink``),
  an output gate per head (``g``), ``o``. A layer with ``kv_from`` has no ``dkv`` and reads that layer's cache unit;
* ``general_delta``: a matrix state per head that decays per key channel and removes along the unit key before it writes
  (``r``, ``k``, ``v``, the decay ``w1``, ``w2``, ``w0``, the removal rate ``a`` with ``a.b``, the head norm's weight ``norm``, the
  output gate ``g``, ``o``).

The feed-forward is a mixture of experts (``l<i>.mlp.router``, ``.correction``, ``.e<j>.{gate,up,down}``) with sigmoid scores, a
choice that a correction steers and groups restrict, and weights that are the chosen scores themselves. ``final.norm`` comes
before the head ``head``. Linear weights are stored ``[out, in]``.
"""
from __future__ import annotations

import math

from levanter_amd.config.tativik import TativikConfig
from levanter_amd.parts.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry, TensorSpec

DECAY_SHARPNESS = math.exp(-0.5)  # w = exp(-DECAY_SHARPNESS * sigmoid(.))
UNIT_KEY_EPS = 1e-6  # u = k / sqrt(sum(k^2) + UNIT_KEY_EPS)
GROUP_SCORE_TOP = 2  # a group of experts is scored by the sum of its two largest choice scores


def tativik_model_spec(cfg: TativikConfig) -> ModelSpec:
    d, eps, groups = cfg.width, float(cfg.norm_eps), int(cfg.norm_groups)
    lin = 1.0 / math.sqrt(d)

    def norm(name: str) -> PartSpec:
        return PartSpec("group_rmsnorm", {"dim": d, "groups": groups, "eps": eps}, {"weight": TensorSpec(name, (d,), init="one_plus_normal", std=0.1)},
                        family="norm")

    def connection(post: str, gate: str) -> PartSpec:
        return PartSpec("gated_post_norm", {"dim": d, "groups": groups, "eps": eps, "mult": float(cfg.residual_mult), "gate": True},
                        {"weight": TensorSpec(post, (d,), init="one_plus_normal", std=0.1), "gate.weight": TensorSpec(gate, (d, d), std=lin),
                         "gate.bias": TensorSpec(f"{gate}.b", (d,), std=0.5)}, family="stream_mix")

    # what a layer's cache unit keeps: the largest window among the layer and the layers that read its unit
    def window_of(m: dict):
        return (m.get("mask") or {}).get("size")

    cache_window = {}
    for i, layer in enumerate(cfg.layers):
        if layer["type"] != "latent_attention":
            continue
        owner = layer["mixer"].get("kv_from")
        owner = i if owner is None else owner
        w = window_of(layer["mixer"])
        if owner not in cache_window:
            cache_window[owner] = w
        elif cache_window[owner] is not None:
            cache_window[owner] = None if w is None else max(w, cache_window[owner])

    def latent(p: str, m: dict, i: int) -> PartSpec:
        H, dk, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        src = m.get("kv_from")
        rot = m.get("rot")
        tensors = {"q_down.weight": TensorSpec(f"{p}.dq", (Q, d), std=lin),
                   "q_norm.weight": TensorSpec(f"{p}.dq.norm", (Q,), init="one_plus_normal", std=0.1),
                   "q.weight": TensorSpec(f"{p}.uq", (H * (dk + dr), Q), std=1.0 / math.sqrt(Q)),
                   "up_k.weight": TensorSpec(f"{p}.uk", (H * dk, R), std=1.0 / math.sqrt(R)),
                   "up_v.weight": TensorSpec(f"{p}.uv", (H * dv, R), std=1.0 / math.sqrt(R)),
                   "sinks": TensorSpec(f"{p}.sink", (H,), std=1.0),
                   "gate.weight": TensorSpec(f"{p}.g", (H, d), std=lin),
                   "out.weight": TensorSpec(f"{p}.o", (d, H * dv), std=1.0 / math.sqrt(H * dv))}
        if src is None:
            tensors["down.weight"] = TensorSpec(f"{p}.dkv", (R + dr, d), std=lin)
            tensors["latent_norm.weight"] = TensorSpec(f"{p}.dkv.norm", (R,), init="one_plus_normal", std=0.1)
        return PartSpec("latent_attention",
                        {"dim": d, "n_heads": H, "head_dim": dk, "value_dim": dv, "latent_dim": R, "query_latent_dim": Q, "rope_dim": dr,
                         "rotary": None if rot is None or not rot["dims"] else {"dims": rot["dims"], "base": float(rot["base"])},
                         "scale": float(m["scale"]), "norm_eps": eps, "window": window_of(m), "cache_window": cache_window[i if src is None else src],
                         "sinks": True, "gate": True, "shared_kv": src is not None}, tensors, family="mixer")

    def delta(p: str, m: dict) -> PartSpec:
        H, dh = m["heads"], m["dim"]
        C = H * dh
        rank = m.get("decay_rank") or -1
        return PartSpec("general_delta_rule",
                        {"dim": d, "n_heads": H, "head_dim": dh, "decay_rank": rank, "sharpness": DECAY_SHARPNESS, "key_eps": UNIT_KEY_EPS, "norm_eps": eps},
                        {"r.weight": TensorSpec(f"{p}.r", (C, d), std=lin), "k.weight": TensorSpec(f"{p}.k", (C, d), std=lin),
                         "v.weight": TensorSpec(f"{p}.v", (C, d), std=lin), "gate.weight": TensorSpec(f"{p}.g", (C, d), std=lin),
                         "removal.weight": TensorSpec(f"{p}.a", (C, d), std=lin), "removal.bias": TensorSpec(f"{p}.a.b", (C,), std=0.5),
                         "decay_down.weight": TensorSpec(f"{p}.w1", (rank, d), std=lin),
                         "decay_up.weight": TensorSpec(f"{p}.w2", (C, rank), std=1.0 / math.sqrt(max(rank, 1))),
                         "decay_up.bias": TensorSpec(f"{p}.w0", (C,), std=1.0),
                         "norm.weight": TensorSpec(f"{p}.norm", (C,), init="one_plus_normal", std=0.1),
                         "out.weight": TensorSpec(f"{p}.o", (d, C), std=1.0 / math.sqrt(C))}, family="mixer")

    def experts(p: str, mlp: dict) -> PartSpec:
        f, router = mlp["expert"]["ff"], mlp["router"]
        E = router["experts"]
        g = router.get("groups") or {"count": 1, "keep": 1}
        tensors = {"router.weight": TensorSpec(f"{p}.router", (E, d), std=lin), "correction": TensorSpec(f"{p}.correction", (E,), std=0.2)}
        for e in range(E):
            tensors[f"experts.{e}.gate.weight"] = TensorSpec(f"{p}.e{e}.gate", (f, d), std=lin)
            tensors[f"experts.{e}.up.weight"] = TensorSpec(f"{p}.e{e}.up", (f, d), std=lin)
            tensors[f"experts.{e}.down.weight"] = TensorSpec(f"{p}.e{e}.down", (d, f), std=1.0 / math.sqrt(f))
        return PartSpec("routed_experts", {"dim": d, "inner_dim": f, "n_experts": E, "top": router["top"], "n_groups": g["count"], "keep": g["keep"],
                                           "group_top": GROUP_SCORE_TOP, "activation": "silu", "renormalize": False, "correction": True},
                        tensors, family="feed_forward")

    layers, plan, ignored, unit_of = [], [], [], {}
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer["mixer"]
        if layer["type"] == "latent_attention":
            mixer = latent(f"{p}.mix", m, i)
            src = m.get("kv_from")
        else:
            mixer, src = delta(f"{p}.mix", m), None
        parts = {"norm1": norm(f"{p}.norm1"), "mixer": mixer, "connect1": connection(f"{p}.norm1b", f"{p}.rg1")}
        mlp = layer.get("mlp")
        if mlp is not None:
            parts["norm2"] = norm(f"{p}.norm2")
            parts["feed_forward"] = experts(f"{p}.mlp", mlp)
            parts["connect2"] = connection(f"{p}.norm2b", f"{p}.rg2")
        else:  # a file may still hold the second sublayer's norms and gate of a layer that has none
            ignored += [rf"l{i}\.norm2b?", rf"l{i}\.rg2(\.b)?"]
        layers.append(LayerSpec("gated_sandwich", parts))
        if src is None:
            unit_of[i] = len(unit_of)
            plan.append(PlanEntry(layer=i, cache=unit_of[i], writes_cache=True))
        else:  # the layer reads the unit that layer `src` has written earlier in the step
            plan.append(PlanEntry(layer=i, cache=unit_of[src], writes_cache=False))

    embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "dim": d, "position": None, "norm": norm("embed.norm")},
                         {"table": TensorSpec("embed", (cfg.vocab, d), std=1.0)}, family="embedding")
    head = PartSpec("linear_head", {"vocab_size": cfg.vocab, "dim": d}, {"weight": TensorSpec("head", (cfg.vocab, d), std=lin)}, family="head")
    return ModelSpec(
        architecture="tativik",
        vocab_size=cfg.vocab,
        dim=d,
        embedding=embedding,
        layers=layers,
        plan=plan,
        final_norm=norm("final.norm"),
        head=head,
        max_positions=None,
        ignored_tensors=tuple(ignored),
        init_std=cfg.initializer_range,
    )
