"""Kegetar, stated plainly: whole sequences in float64, one function per mechanism, no cache, no kernels, nothing shared
with the package. ``weights`` maps checkpoint tensor names to float64 tensors, ``cfg`` is the raw config.json dict.

Notation: x the residual stream ``[T, D]``, h a sublayer's input (x itself: the norms stand behind the sublayers),
positions count from 0.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

F64 = torch.float64

GELU_C = math.sqrt(2.0 / math.pi)
EXPERT_SIGMOID_SLOPE = 1.702


# ---- norms ------------------------------------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension, times w."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def one_plus_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The norm of the residual stream: its weight is stored as the distance from one."""
    return rms_norm(x, 1.0 + w, eps)


# ---- embedding --------------------------------------------------------------------------------------------------
def bigram_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the pair table for each token: a hash of (token before, token); the sequence's first token takes the last row."""
    return [buckets if t == 0 else (tokens[t - 1] * mul_prev + tokens[t] * mul_cur) % buckets for t in range(len(tokens))]


def embed(tokens: List[int], weights: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    x = weights["embed"][torch.tensor(tokens)]
    b = (cfg.get("embedding") or {}).get("bigram")
    if b:
        x = x + weights["bigram"][torch.tensor(bigram_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"]))]
    return x


# ---- positions --------------------------------------------------------------------------------------------------
def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]) -> Tuple[List[float], float]:
    """Angle per position of each of the dims/2 pairs, and the factor on cosine and sine. Without scaling: base^(-2i/dims)
    and 1. With (factor, original, fast, slow): a pair index i is placed on a ramp between the index whose wavelength fits
    ``fast`` times into the original length and the one that fits ``slow`` times; below the ramp the frequency stays, above it
    is divided by the factor, on it the two are mixed linearly."""
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, original, fast, slow = (float(scaling[k]) for k in ("factor", "original", "fast", "slow"))

    def index_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_pairs(v: torch.Tensor, positions: torch.Tensor, freqs: List[float], magnitude: float) -> torch.Tensor:
    """v ``[T, heads, n]``: dimensions (2i, 2i+1), i < len(freqs), turn by p * freqs[i], cosine and sine both times ``magnitude``;
    dimensions from 2 len(freqs) on pass unchanged."""
    out = v.clone()
    n = len(freqs)
    if n == 0:
        return out
    a = positions.to(F64)[:, None] * torch.tensor(freqs, dtype=F64)[None, :]
    cos, sin = (torch.cos(a) * magnitude)[:, None, :], (torch.sin(a) * magnitude)[:, None, :]
    u, w = v[..., 0:2 * n:2], v[..., 1:2 * n:2]
    out[..., 0:2 * n:2] = u * cos - w * sin
    out[..., 1:2 * n:2] = w * cos + u * sin
    return out


# ---- visibility -------------------------------------------------------------------------------------------------
def visible(T: int, size: Optional[int], keep_first: int = 0) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff j <= i and (i - j < size or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & ((i - j < size) | (j < keep_first))
    return ok


def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, see: torch.Tensor,
                      slopes: Optional[List[float]] = None) -> torch.Tensor:
    """q ``[T, H, d]``, k ``[T, G, d]``, v ``[T, G, dv]`` -> ``[T, H, dv]``; head h reads key/value head h // (H / G); score
    scale q.k - slope_h (i - j) over the visible keys."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if slopes is not None:
            s = s - slopes[h] * dist
        s = s.masked_fill(~see, -math.inf)
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


def distance_slopes(H: int) -> List[float]:
    return [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]


# ---- the mixers -------------------------------------------------------------------------------------------------
def rotary_gated_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Windowed attention that keeps the first tokens in sight: per-head RMS norm of q and k with one weight for all heads,
    rotation of pairs, softmax, an element-wise sigmoid gate from the same input, output projection."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[f"{p}.q"].T).view(T, H, d)
    k = (h @ W[f"{p}.k"].T).view(T, G, d)
    v = (h @ W[f"{p}.v"].T).view(T, G, dv)
    q = rms_norm(q, W[f"{p}.q.norm"], eps)
    k = rms_norm(k, W[f"{p}.k.norm"], eps)
    rot = m.get("rot")
    pos = torch.arange(T)
    if rot and rot.get("dims"):
        freqs, mag = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_pairs(q, pos, freqs, mag), rotate_pairs(k, pos, freqs, mag)
    mask = m.get("mask") or {}
    o = softmax_attention(q, k, v, m["scale"], visible(T, mask.get("size"), mask.get("keep_first", 0)))
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ W[f"{p}.g"].T)
    return o @ W[f"{p}.o"].T


def gated_linear_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                           state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """A matrix state per head, S <- diag(alpha) S + k v^T, read as S^T q; alpha = sigmoid(low-rank map)^(1 / tau) per key
    channel. Returns the output and the final state ``[H, d, dv]``."""
    T = h.shape[0]
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    q = (h @ W[f"{p}.q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[f"{p}.k"].T).view(T, H, d)
    v = (h @ W[f"{p}.v"].T).view(T, H, dv)
    z = (h @ W[f"{p}.a1"].T) @ W[f"{p}.a2"].T + W[f"{p}.a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(T, H, d)
    S = torch.zeros(H, d, dv, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hij,hi->hj", S, q[t])
    o = rms_norm(o, W[f"{p}.norm"], eps).reshape(T, H * dv)
    g = h @ W[f"{p}.g"].T
    return (o * g * torch.sigmoid(g)) @ W[f"{p}.o"].T, S


def parallel_mixer(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Half the sum of the two branches, each through an RMS norm of the model's width with a weight of its own."""
    left = rotary_gated_attention(h, W, f"{p}.left", m["left"], eps)
    right, _ = gated_linear_attention(h, W, f"{p}.right", m["right"], eps)
    return 0.5 * (rms_norm(left, W[f"{p}.left.out"], eps) + rms_norm(right, W[f"{p}.right.out"], eps))


def keys_as_values_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Attention without a value projection: the keys as projected are the values; q and k are normed over the whole
    projection; positions enter as a distance term only."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = h @ W[f"{p}.q"].T + W[f"{p}.q.b"]
    k = h @ W[f"{p}.k"].T + W[f"{p}.k.b"]
    v = k.view(T, G, d)
    q = rms_norm(q, W[f"{p}.q.norm"], eps).view(T, H, d)
    k = rms_norm(k, W[f"{p}.k.norm"], eps).view(T, G, d)
    size = (m.get("mask") or {}).get("size")
    o = softmax_attention(q, k, v, m["scale"], visible(T, size), distance_slopes(H))
    return o.reshape(T, H * d) @ W[f"{p}.o"].T


# ---- feed-forwards ----------------------------------------------------------------------------------------------
def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(GELU_C * (z + 0.044715 * z ** 3)))


def dense_feed_forward(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    g = h @ W[f"{p}.gate"].T + W[f"{p}.gate.b"]
    u = h @ W[f"{p}.up"].T + W[f"{p}.up.b"]
    return (gelu_tanh(g) * u) @ W[f"{p}.down"].T + W[f"{p}.down.b"]


def clamped_expert(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, limit: float) -> torch.Tensor:
    g = (h @ W[f"{p}.gate"].T).clamp(max=limit)
    u = (h @ W[f"{p}.up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(EXPERT_SIGMOID_SLOPE * g) * (u + 1.0)) @ W[f"{p}.down"].T


def route(z: torch.Tensor, correction: torch.Tensor, top: int, n_groups: int, keep: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """z ``[T, N]`` router logits (identity experts included). Returns the chosen indices ``[T, top]``, their weights and the
    margin by which each token's choice was decided (smallest gap between a winner and the best loser, among groups too)."""
    T, N = z.shape
    s = torch.softmax(z, -1)
    c = s + correction
    per = N // n_groups
    group_score = c.view(T, n_groups, per).max(-1).values
    order = torch.argsort(group_score, dim=-1, descending=True, stable=True)
    allowed = torch.zeros(T, n_groups, dtype=torch.bool)
    allowed.scatter_(1, order[:, :keep], True)
    margin = torch.full((T,), math.inf, dtype=F64)
    if keep < n_groups:
        gs = torch.gather(group_score, 1, order)
        margin = torch.minimum(margin, gs[:, keep - 1] - gs[:, keep])
    masked = c.masked_fill(~allowed[:, :, None].expand(T, n_groups, per).reshape(T, N), -math.inf)
    eorder = torch.argsort(masked, dim=-1, descending=True, stable=True)
    chosen = eorder[:, :top]
    if top < N:
        es = torch.gather(masked, 1, eorder)
        gap = es[:, top - 1] - es[:, top]
        margin = torch.minimum(margin, torch.where(torch.isfinite(gap), gap, torch.full_like(gap, math.inf)))
    return chosen, torch.gather(s, 1, chosen), margin


def expert_feed_forward(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, mlp: dict) -> Tuple[torch.Tensor, torch.Tensor]:
    """Routed experts (the last ``identity`` router outputs stand for experts that return their input), weights not
    renormalised, plus a shared expert for every token. Returns the result and the routing margins."""
    r = mlp["router"]
    E, ident, top = r["experts"], r.get("identity", 0), r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    z = h @ W[f"{p}.router"].T
    chosen, weight, margin = route(z, W[f"{p}.correction"], top, groups["count"], groups["keep"])
    limit = float(mlp["expert"]["limit"])
    y = torch.zeros_like(h)
    outs = {}
    for t in range(h.shape[0]):
        for c in range(top):
            e = int(chosen[t, c])
            if e >= E:
                y[t] += weight[t, c] * h[t]
            else:
                if e not in outs:
                    outs[e] = clamped_expert(h, W, f"{p}.e{e}", limit)
                y[t] += weight[t, c] * outs[e][t]
    shared = mlp.get("shared")
    if shared:
        y = y + clamped_expert(h, W, f"{p}.shared", float(shared["limit"]))
    return y, margin


# ---- the model --------------------------------------------------------------------------------------------------
def forward(tokens: List[int], weights: Dict[str, torch.Tensor], cfg: dict) -> Tuple[torch.Tensor, List[torch.Tensor], torch.Tensor]:
    """Logits ``[T, vocab]``, the residual stream after every layer run, and the smallest routing margin per token."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = embed(tokens, weights, cfg)
    streams = []
    margin = torch.full((len(tokens),), math.inf, dtype=F64)
    for i, layer in enumerate(cfg["layers"]):
        owner = i
        while cfg["layers"][owner].get("weights_of") is not None:  # whose tensors the layer runs
            owner = cfg["layers"][owner]["weights_of"]
        p = f"l{owner}"
        m = layer["mixer"]
        if layer["type"] == "parallel":
            y = parallel_mixer(x, weights, f"{p}.mix", m, eps)
        else:
            y = keys_as_values_attention(x, weights, f"{p}.mix", m, eps)
        x = x + mult * one_plus_norm(y, weights[f"{p}.norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                y = dense_feed_forward(x, weights, f"{p}.mlp")
            else:
                y, mg = expert_feed_forward(x, weights, f"{p}.mlp", mlp)
                margin = torch.minimum(margin, mg)
            x = x + mult * one_plus_norm(y, weights[f"{p}.norm2"], eps)
        streams.append(x.clone())
    hfin = one_plus_norm(x, weights["final.norm"], eps)
    return hfin @ weights["head"].T, streams, margin


def plain_logits(W: Dict[str, torch.Tensor], cfg: dict, tokens) -> torch.Tensor:
    return forward([int(t) for t in tokens], W, cfg)[0]


def plain_greedy(W: Dict[str, torch.Tensor], cfg: dict, prompt: List[int], n_new: int) -> List[int]:
    toks = [int(t) for t in prompt]
    for _ in range(n_new):
        toks.append(int(torch.argmax(plain_logits(W, cfg, toks)[-1])))
    return toks[len(prompt):]


# ---- configurations and weights for tests -----------------------------------------------------------------------
def left_sizes(heads=4, kv_heads=2, dim=16, vdim=8, window=24, keep_first=3, rot_dims=None, base=10000.0, scaling="default", scale=None) -> dict:
    if scaling == "default":
        scaling = {"factor": 3.0, "original": 40, "fast": 8.0, "slow": 1.0}
    rot = None if rot_dims == 0 else {"dims": dim if rot_dims is None else rot_dims, "base": base, **({"scaling": scaling} if scaling else {})}
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale}
    if rot:
        m["rot"] = rot
    if window is not None:
        m["mask"] = {"size": window, "keep_first": keep_first}
    return m


def right_sizes(heads=2, dim=16, vdim=8, tau=8.0, decay_rank=4) -> dict:
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": decay_rank}


def parallel_layer(left=None, right=None, mlp="dense", weights_of=None) -> dict:
    L = {"type": "parallel", "mixer": {"left": left or left_sizes(), "right": right or right_sizes()}, "mlp": dense_mlp() if mlp == "dense" else mlp}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def attention_layer(heads=4, kv_heads=1, dim=16, window=20, scale=None, mlp="dense", weights_of=None) -> dict:
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5 if scale is None else scale}
    if window is not None:
        m["mask"] = {"size": window}
    L = {"type": "attention", "mixer": m, "mlp": dense_mlp() if mlp == "dense" else mlp}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def dense_mlp(ff=48) -> dict:
    return {"kind": "dense", "ff": ff}


def experts_mlp(ff=24, experts=6, top=2, identity=2, groups=(2, 1), limit=2.0, shared=32, shared_limit=1.5) -> dict:
    router = {"experts": experts, "top": top, "identity": identity}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}
    if shared:
        mlp["shared"] = {"ff": shared, "limit": shared_limit}
    return mlp


def make_config(vocab=97, width=64, layers=None, eps=1e-5, mult=0.6, bigram=(31, 5, 3)) -> dict:
    cfg = {"architecture": "Kegetar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
           "layers": layers if layers is not None else [parallel_layer(), attention_layer()]}
    if bigram:
        cfg["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return cfg


def random_weights(cfg: dict, seed: int, dtype=F64, clear_routing: bool = False) -> Dict[str, torch.Tensor]:
    """Weights drawn so that every mechanism matters: scores of order one, gates that are not saturated, decays over a wide
    range, activations that reach their limits, router scores whose order the correction changes. Values are bfloat16 numbers
    (a file stores them exactly). ``clear_routing``: routers that decide by a wide margin (scores that move little with the
    input, corrections a fixed step apart in a random order), for runs in 16-bit arithmetic, where a choice by less than the
    inputs' rounding could fall either way."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16).to(dtype)

    W = {"embed": rn(V, D), "final.norm": rn(D, std=0.2), "head": rn(V, D, std=1 / math.sqrt(D))}
    b = (cfg.get("embedding") or {}).get("bigram")
    if b:
        W["bigram"] = rn(b["buckets"] + 1, D, std=0.7)
    lin = 1 / math.sqrt(D)
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        m, p = L["mixer"], f"l{i}."
        W[p + "norm1"] = rn(D, std=0.2)
        if L["type"] == "parallel":
            le, ri = m["left"], m["right"]
            H, G, dk, dv = le["heads"], le["kv_heads"], le["dim"], le["vdim"]
            q = p + "mix.left."
            W[q + "q"], W[q + "k"], W[q + "v"] = rn(H * dk, D, std=lin), rn(G * dk, D, std=lin), rn(G * dv, D, std=lin)
            W[q + "q.norm"], W[q + "k.norm"] = 1.5 + rn(dk, std=0.3), 1.5 + rn(dk, std=0.3)
            W[q + "g"] = rn(H * dv, D, std=1.5 * lin)
            W[q + "o"] = rn(D, H * dv, std=1 / math.sqrt(H * dv))
            W[p + "mix.left.out"] = 1 + rn(D, std=0.2)
            H, dk, dv, rank = ri["heads"], ri["dim"], ri["vdim"], ri["decay_rank"]
            q = p + "mix.right."
            W[q + "q"], W[q + "k"] = rn(H * dk, D, std=lin), rn(H * dk, D, std=lin)
            W[q + "v"], W[q + "g"] = rn(H * dv, D, std=lin), rn(H * dv, D, std=1.5 * lin)
            W[q + "a1"] = rn(rank, D, std=lin)
            W[q + "a2"] = rn(H * dk, rank, std=2 / math.sqrt(rank))
            W[q + "a2.b"] = rn(H * dk, std=2.0)
            W[q + "norm"] = 1 + rn(dv, std=0.2)
            W[q + "o"] = rn(D, H * dv, std=1 / math.sqrt(H * dv))
            W[p + "mix.right.out"] = 1 + rn(D, std=0.2)
        else:
            H, G, dk = m["heads"], m["kv_heads"], m["dim"]
            q = p + "mix."
            W[q + "q"], W[q + "q.b"] = rn(H * dk, D, std=lin), rn(H * dk, std=0.3)
            W[q + "k"], W[q + "k.b"] = rn(G * dk, D, std=lin), rn(G * dk, std=0.3)
            W[q + "q.norm"], W[q + "k.norm"] = 1.5 + rn(H * dk, std=0.3), 1.5 + rn(G * dk, std=0.3)
            W[q + "o"] = rn(D, H * dk, std=1 / math.sqrt(H * dk))
        mlp = L.get("mlp")
        if mlp is None:
            continue
        W[p + "norm2"] = rn(D, std=0.2)
        q = p + "mlp."
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            W[q + "gate"], W[q + "gate.b"] = rn(F, D, std=lin), rn(F, std=0.3)
            W[q + "up"], W[q + "up.b"] = rn(F, D, std=lin), rn(F, std=0.3)
            W[q + "down"], W[q + "down.b"] = rn(D, F, std=1 / math.sqrt(F)), rn(D, std=0.3)
            continue
        F, r = mlp["expert"]["ff"], mlp["router"]
        E, N = r["experts"], r["experts"] + r.get("identity", 0)
        W[q + "router"] = rn(N, D, std=(0.002 if clear_routing else 0.15) * lin)  # the router reads the stream itself, whose entries are of order ten
        W[q + "correction"] = rn(N, std=0.1)
        if clear_routing:
            W[q + "correction"] = (torch.randperm(N, generator=g).to(torch.float32) * 0.0625 - 0.25).to(torch.bfloat16).to(dtype)
        for e in range(E):
            W[q + f"e{e}.gate"], W[q + f"e{e}.up"] = rn(F, D, std=2 * lin), rn(F, D, std=2 * lin)
            W[q + f"e{e}.down"] = rn(D, F, std=1 / math.sqrt(F))
        sh = mlp.get("shared")
        if sh:
            W[q + "shared.gate"], W[q + "shared.up"] = rn(sh["ff"], D, std=2 * lin), rn(sh["ff"], D, std=2 * lin)
            W[q + "shared.down"] = rn(D, sh["ff"], std=1 / math.sqrt(sh["ff"]))
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
        if L["type"] == "parallel":
            L["mixer"]["right"].pop("decay_rank", None)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(out, f)
    save_file({k: v.to(dtype).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return path


def first_close_call(W: Dict[str, torch.Tensor], cfg: dict, tokens, delta: float) -> int:
    """The first position at which some router decides by less than ``delta`` (the number of tokens if there is none)."""
    margin = forward([int(t) for t in tokens], W, cfg)[2]
    close = (margin < delta).nonzero()
    return int(close[0]) if close.numel() else len(tokens)
