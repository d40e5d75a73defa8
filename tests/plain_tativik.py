"""Tativik, stated plainly: whole sequences in float64, one function per mechanism, no cache, no kernels, nothing shared
with the package. ``weights`` maps checkpoint tensor names to float64 tensors, ``cfg`` is the raw config.json dict.

Notation: x the residual stream ``[T, D]``, h a sublayer's input, positions count from 0.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

F64 = torch.float64


# ---- norms ------------------------------------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension, times w."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def group_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """The last dimension in ``groups`` equal consecutive parts, each divided by its own root mean square; then times w."""
    T, D = x.shape
    parts = x.view(T, groups, D // groups)
    return rms_norm(parts, None, eps).reshape(T, D) * w


# ---- positions --------------------------------------------------------------------------------------------------
def rotate_half(v: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """v ``[T, ..., n]``: dimension i < dims/2 is paired with i + dims/2 and the pair turned by p * base^(-2i/dims); dimensions
    from ``dims`` on pass unchanged."""
    half = dims // 2
    out = v.clone()
    if half == 0:
        return out
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = positions.to(F64)[:, None] * f[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    cos, sin = torch.cos(a).view(shape), torch.sin(a).view(shape)
    lo, hi = v[..., :half], v[..., half:dims]
    out[..., :half] = lo * cos - hi * sin
    out[..., half:dims] = hi * cos + lo * sin
    return out


def window_visible(T: int, size: Optional[int]) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff 0 <= i - j < size (no size: every j <= i)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & (i - j < size)
    return ok


def softmax_with_sink(scores: torch.Tensor, visible: torch.Tensor, sink: Optional[torch.Tensor]) -> torch.Tensor:
    """scores ``[H, T, T]``; weights over the visible keys whose denominator also holds exp(sink_h), once per row."""
    s = scores.masked_fill(~visible[None], -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink.view(-1, 1, 1))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.view(-1, 1, 1) - m)
    return e / den


# ---- latent attention ---------------------------------------------------------------------------------------------
def latent_kv(h: torch.Tensor, w_dkv: torch.Tensor, norm_w: torch.Tensor, kv_rank: int, eps: float, rot_dims: int, base: float
              ) -> Tuple[torch.Tensor, torch.Tensor]:
    """What a layer caches: the normed latent ``[T, kv_rank]`` and the rotated key part ``[T, rot_dim]`` that all heads share."""
    d = h @ w_dkv.T
    c = rms_norm(d[:, :kv_rank], norm_w, eps)
    k_rot = rotate_half(d[:, kv_rank:], torch.arange(h.shape[0]), rot_dims, base)
    return c, k_rot


def latent_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                     kv: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> Tuple[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """The mixer's output ``[T, D]`` and the (latent, rotated key part) it used: its own, or ``kv`` of the layer it borrows from."""
    T = h.shape[0]
    H, dk, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    rot_dims, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
    cq = rms_norm(h @ W[f"{p}.dq"].T, W[f"{p}.dq.norm"], eps)
    q = (cq @ W[f"{p}.uq"].T).view(T, H, dk + dr)
    q_plain = q[..., :dk]
    q_rot = rotate_half(q[..., dk:], torch.arange(T), rot_dims, base)
    if kv is None:
        kv = latent_kv(h, W[f"{p}.dkv"], W[f"{p}.dkv.norm"], R, eps, rot_dims, base)
    c, k_rot = kv
    k_plain = (c @ W[f"{p}.uk"].T).view(T, H, dk)
    v = (c @ W[f"{p}.uv"].T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * float(m["scale"])
    size = (m.get("mask") or {}).get("size")
    weights = softmax_with_sink(scores, window_visible(T, size), W.get(f"{p}.sink"))
    o = torch.einsum("hij,jhd->ihd", weights, v)
    o = o * torch.sigmoid(h @ W[f"{p}.g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[f"{p}.o"].T, kv


# ---- generalized delta rule ---------------------------------------------------------------------------------------
DECAY_SHARPNESS = math.exp(-0.5)
UNIT_KEY_EPS = 1e-6


def delta_rule_scan(r, k, v, w, a, state=None):
    """Per head: S <- diag(w_t) S - (a_t * u_t)(u_t^T S) + k_t v_t^T with u = k / sqrt(sum(k^2) + 1e-6), both terms reading the old
    S; o_t = S^T r_t. All ``[T, H, d]``; returns o ``[T, H, d]`` and the last state ``[H, d, d]`` (key channel, value channel)."""
    T, H, d = k.shape
    S = torch.zeros(H, d, d, dtype=F64) if state is None else state.clone()
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + UNIT_KEY_EPS)
    out = torch.empty(T, H, d, dtype=F64)
    for t in range(T):
        uS = torch.einsum("hi,hij->hj", u[t], S)
        S = w[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hij,hi->hj", S, r[t])
    return out, S


def general_delta(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r, k, v = ((h @ W[f"{p}.{n}"].T).view(T, H, d) for n in ("r", "k", "v"))
    w = torch.exp(-DECAY_SHARPNESS * torch.sigmoid(torch.tanh(h @ W[f"{p}.w1"].T) @ W[f"{p}.w2"].T + W[f"{p}.w0"])).view(T, H, d)
    a = torch.sigmoid(h @ W[f"{p}.a"].T + W[f"{p}.a.b"]).view(T, H, d)
    o, _ = delta_rule_scan(r, k, v, w, a)
    o = rms_norm(o, None, eps).reshape(T, H * d) * W[f"{p}.norm"]
    o = o * torch.sigmoid(h @ W[f"{p}.g"].T)
    return o @ W[f"{p}.o"].T


# ---- mixture of experts -------------------------------------------------------------------------------------------
def route(z: torch.Tensor, correction: torch.Tensor, top: int, n_groups: int, keep: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """z ``[T, E]`` router logits. Returns the chosen experts ``[T, top]`` and their weights: s = sigmoid(z); the choice goes by
    s + correction among the experts of the ``keep`` groups whose two largest choice scores sum highest; the weights are s."""
    T, E = z.shape
    s = torch.sigmoid(z)
    choice = s + correction
    per = E // n_groups
    grouped = choice.view(T, n_groups, per)
    group_score = grouped.topk(min(2, per), -1).values.sum(-1)
    kept = group_score.topk(keep, -1).indices
    allowed = torch.zeros(T, n_groups, dtype=torch.bool).scatter_(1, kept, True)
    masked = choice.masked_fill(~allowed[:, :, None].expand(T, n_groups, per).reshape(T, E), -math.inf)
    chosen = masked.topk(top, -1).indices
    return chosen, s.gather(1, chosen)


def expert(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    g = h @ W[f"{p}.gate"].T
    return ((g * torch.sigmoid(g)) * (h @ W[f"{p}.up"].T)) @ W[f"{p}.down"].T


def route_margin(z: torch.Tensor, correction: torch.Tensor, top: int, n_groups: int, keep: int) -> torch.Tensor:
    """Per token, how far the router's choice is from another one: the gap in choice score between the last expert taken and
    the best one left out, and between the last group kept and the best one dropped; infinite where there is no choice."""
    T, E = z.shape
    choice = torch.sigmoid(z) + correction
    per = E // n_groups
    out = torch.full((T,), math.inf, dtype=F64)
    group_score = choice.view(T, n_groups, per).topk(min(2, per), -1).values.sum(-1)
    allowed = torch.ones(T, n_groups, dtype=torch.bool)
    if keep < n_groups:
        best = group_score.topk(keep + 1, -1)
        out = torch.minimum(out, best.values[:, keep - 1] - best.values[:, keep])
        allowed = torch.zeros(T, n_groups, dtype=torch.bool).scatter_(1, best.indices[:, :keep], True)
    if top < keep * per:
        masked = choice.masked_fill(~allowed[:, :, None].expand(T, n_groups, per).reshape(T, E), -math.inf)
        best = masked.topk(top + 1, -1).values
        out = torch.minimum(out, best[:, top - 1] - best[:, top])
    return out


def moe(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, mlp: dict, margins: Optional[list] = None) -> torch.Tensor:
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weights = route(h @ W[f"{p}.router"].T, W[f"{p}.correction"], r["top"], groups["count"], groups["keep"])
    if margins is not None:
        margins.append(route_margin(h @ W[f"{p}.router"].T, W[f"{p}.correction"], r["top"], groups["count"], groups["keep"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t].tolist(), weights[t]):
            out[t] += wt * expert(h[t:t + 1], W, f"{p}.e{e}")[0]
    return out


# ---- the model ----------------------------------------------------------------------------------------------------
def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False, margins: Optional[list] = None):
    """Logits ``[T, vocab]`` of one whole sequence (and the residual stream after every layer). ``margins``: a list that takes
    every routed layer's ``route_margin``."""
    eps, groups, mult = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"]), float(cfg["residual_mult"])

    def norm(x, name):
        return group_rms_norm(x, W[name], groups, eps)

    x = norm(W["embed"][torch.tensor(tokens)], "embed.norm")
    kept: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        h = norm(x, f"{p}.norm1")
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            y, kv = latent_attention(h, W, f"{p}.mix", m, eps, None if src is None else kept[src])
            if src is None:
                kept[i] = kv
        elif layer["type"] == "general_delta":
            y = general_delta(h, W, f"{p}.mix", m, eps)
        else:
            raise ValueError(layer["type"])
        y = y * torch.sigmoid(h @ W[f"{p}.rg1"].T + W[f"{p}.rg1.b"])
        x = x + mult * norm(y, f"{p}.norm1b")
        if layer.get("mlp") is not None:
            h = norm(x, f"{p}.norm2")
            y = moe(h, W, f"{p}.mlp", layer["mlp"], margins)
            y = y * torch.sigmoid(h @ W[f"{p}.rg2"].T + W[f"{p}.rg2.b"])
            x = x + mult * norm(y, f"{p}.norm2b")
        after.append(x)
    logits = norm(x, "final.norm") @ W["head"].T
    return (logits, torch.stack(after)) if return_layers else logits


def plain_logits(W: Dict[str, torch.Tensor], cfg: dict, tokens) -> torch.Tensor:
    return forward(cfg, W, [int(t) for t in tokens])


def first_close_call(W: Dict[str, torch.Tensor], cfg: dict, tokens, delta: float) -> int:
    """The first position at which some layer's router decides by less than ``delta`` (the sequence's length if none does). In
    16-bit arithmetic such a choice may fall the other way: that token's result is then another model's, and so is, through
    caches and states, every later token's. Nothing that a test asserts may rest on such a position."""
    margins: list = []
    forward(cfg, W, [int(t) for t in tokens], margins=margins)
    if not margins:
        return len(tokens)
    close = (torch.stack(margins).min(0).values < delta).nonzero().flatten()
    return int(close[0]) if close.numel() else len(tokens)


def plain_greedy(W: Dict[str, torch.Tensor], cfg: dict, prompt: List[int], n_new: int) -> List[int]:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(cfg, W, toks)[-1])))
    return toks[len(prompt):]


# ---- small configurations and weights for the tests ---------------------------------------------------------------------
def latent_layer(heads=4, dim=16, rot_dim=8, vdim=8, kv_rank=24, q_rank=16, window=None, rot_dims=None, base=10000.0, scale=None, kv_from=None,
                 mlp="default") -> dict:
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)}
    if rot_dim:
        m["rot"] = {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}
    if window is not None:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": experts_mlp() if mlp == "default" else mlp}


def delta_layer(heads=2, dim=16, decay_rank=8, mlp="default") -> dict:
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim, "decay_rank": decay_rank}, "mlp": experts_mlp() if mlp == "default" else mlp}


def experts_mlp(ff=24, experts=8, top=2, groups=None) -> dict:
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def make_config(vocab=97, width=64, layers=None, eps=1e-5, groups=2, mult=0.7) -> dict:
    return {"architecture": "Tativik", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups}, "residual_mult": mult, "layers": layers}


def random_weights(cfg: dict, seed: int, dtype=F64, clear_routing: bool = False) -> Dict[str, torch.Tensor]:
    """Weights drawn so that every mechanism matters: scores of order one, sinks that take a visible share of the weight,
    gates that are not saturated, decays and removal rates over their whole range, router scores whose order the correction
    changes. Values are bfloat16 numbers (a file stores them exactly). ``clear_routing``: routers that decide by a wide margin
    (scores near one half that move a little with the input, corrections drawn until every border of the choice has a wide gap), for runs in 16-bit
    arithmetic, where a choice by less than the inputs' rounding could fall either way."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16).to(dtype)

    W = {"embed": rn(V, D), "embed.norm": 1 + rn(D, std=0.2), "final.norm": 1 + rn(D, std=0.2), "head": rn(V, D, std=1 / math.sqrt(D))}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], f"l{i}."
        for n in ("norm1", "norm1b"):
            W[p + n] = 1 + rn(D, std=0.2)
        W[p + "rg1"] = rn(D, D, std=1 / math.sqrt(D))
        W[p + "rg1.b"] = rn(D, std=0.5)
        if L["type"] == "latent_attention":
            H, dk, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            W[p + "mix.dq"] = rn(Q, D, std=1 / math.sqrt(D))
            W[p + "mix.dq.norm"] = 1 + rn(Q, std=0.2)
            W[p + "mix.uq"] = rn(H * (dk + dr), Q, std=1.5 / math.sqrt(Q))
            if m.get("kv_from") is None:
                W[p + "mix.dkv"] = rn(R + dr, D, std=1.5 / math.sqrt(D))
                W[p + "mix.dkv.norm"] = 1 + rn(R, std=0.2)
            W[p + "mix.uk"] = rn(H * dk, R, std=1.5 / math.sqrt(R))
            W[p + "mix.uv"] = rn(H * dv, R, std=1 / math.sqrt(R))
            W[p + "mix.sink"] = rn(H, std=1.5)
            W[p + "mix.g"] = rn(H, D, std=1.5 / math.sqrt(D))
            W[p + "mix.o"] = rn(D, H * dv, std=1 / math.sqrt(H * dv))
        else:
            H, d, rank = m["heads"], m["dim"], m["decay_rank"]
            C = H * d
            for n in ("r", "k", "v", "g", "a"):
                W[p + f"mix.{n}"] = rn(C, D, std=1 / math.sqrt(D))
            W[p + "mix.a.b"] = rn(C, std=1.0)
            W[p + "mix.w1"] = rn(rank, D, std=1 / math.sqrt(D))
            W[p + "mix.w2"] = rn(C, rank, std=2 / math.sqrt(rank))
            W[p + "mix.w0"] = rn(C, std=1.5)
            W[p + "mix.norm"] = 1 + rn(C, std=0.2)
            W[p + "mix.o"] = rn(D, C, std=1 / math.sqrt(C))
        mlp = L.get("mlp")
        if mlp is not None:
            F, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            for n in ("norm2", "norm2b"):
                W[p + n] = 1 + rn(D, std=0.2)
            W[p + "rg2"] = rn(D, D, std=1 / math.sqrt(D))
            W[p + "rg2.b"] = rn(D, std=0.5)
            W[p + "mlp.router"] = rn(E, D, std=(0.05 if clear_routing else 1.5) / math.sqrt(D))
            W[p + "mlp.correction"] = rn(E, std=0.3)
            while clear_routing:  # corrections that leave a wide gap at every border of the choice, between groups too
                corr = (torch.rand(E, generator=g) * 0.3 * E - 0.5).to(torch.bfloat16).to(dtype)
                r = mlp["router"]
                gr = r.get("groups") or {"count": 1, "keep": 1}
                if float(route_margin(torch.zeros(1, E, dtype=dtype), corr, r["top"], gr["count"], gr["keep"])[0]) >= 0.15:
                    W[p + "mlp.correction"] = corr
                    break
            for e in range(E):
                W[p + f"mlp.e{e}.gate"] = rn(F, D, std=1 / math.sqrt(D))
                W[p + f"mlp.e{e}.up"] = rn(F, D, std=1 / math.sqrt(D))
                W[p + f"mlp.e{e}.down"] = rn(D, F, std=1 / math.sqrt(F))
    return W


def write_folder(cfg: dict, W: Dict[str, torch.Tensor], path: str, dtype=torch.bfloat16) -> str:
    """config.json and model.safetensors of these weights, through the safetensors package. The inner size of the decay's map
    is left to the tensors: the written configuration does not name it."""
    import copy
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    out = copy.deepcopy(cfg)
    for L in out["layers"]:
        L["mixer"].pop("decay_rank", None)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(out, f)
    save_file({k: v.to(dtype).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return path
