"""Plain torch statements of what each HIP kernel computes, with the kernel library's interface.

Two uses: the GPU tests compare every kernel with the function of the same name here, at sizes
other than the engine's; and the CPU tests install an instance in place of the HIP library so
that the host logic (step function, cache manager, scheduler, trace replay) runs without a GPU.
It is not part of the product: the package never imports it.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch
import torch.nn.functional as F


def _act(name):
    return {
        "none": lambda u: u,
        "gelu": lambda u: F.gelu(u),
        "gelu_new": lambda u: F.gelu(u, approximate="tanh"),
        "relu": F.relu,
        "silu": F.silu,
        "swish": F.silu,
        "quick_gelu": lambda u: u * torch.sigmoid(1.702 * u),
        "tanh": torch.tanh,
        "relu_squared": lambda u: F.relu(u) ** 2,
    }[name]


# ---- Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3") in numpy ----
def philox4x32_10(c0, c1, c2, c3, k0, k1):
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint64) for c in (c0, c1, c2, c3))
    k0 = np.uint64(k0)
    k1 = np.uint64(k1)
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c0
        p1 = np.uint64(0xCD9E8D57) * c2
        n0 = ((p1 >> np.uint64(32)) ^ c1 ^ k0) & mask
        n1 = p1 & mask
        n2 = ((p0 >> np.uint64(32)) ^ c3 ^ k1) & mask
        n3 = p0 & mask
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return c0, c1, c2, c3


def uniform_from_bits(bits: np.ndarray) -> np.ndarray:
    """(top 23 bits + 1/2) / 2^23 in float32: exact, inside (0, 1) at both ends of the range."""
    return ((bits.astype(np.uint32) >> 9).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)


def gumbel_from_bits(bits: np.ndarray) -> np.ndarray:
    u = uniform_from_bits(bits)
    return -np.log(-np.log(u, dtype=np.float32), dtype=np.float32)


def gumbel_noise(key0: int, key1: int, position: int, vocab: int) -> torch.Tensor:
    """The Gumbel noise the sampling kernel adds to entry v: counter (v // 4, position, 0, 0), lane v % 4."""
    groups = (vocab + 3) // 4
    g = np.arange(groups, dtype=np.uint64)
    z = np.zeros(groups, dtype=np.uint64)
    outs = philox4x32_10(g, z + np.uint64(position & 0xFFFFFFFF), z, z, key0 & 0xFFFFFFFF, key1 & 0xFFFFFFFF)
    bits = np.stack(outs, axis=1).reshape(-1)[:vocab].astype(np.uint32)
    return torch.from_numpy(gumbel_from_bits(bits))


class EmulatedKernels:
    path = "<emulated>"

    # ---- embedding
    def embed(self, tokens, positions, table, pos_table, out, scale=1.0) -> None:
        x = table[tokens.long()].float()
        if pos_table is not None:
            x = x + pos_table[positions.long()].float()
        out.copy_(x * scale)

    def pair_embed_add(self, tokens, positions, token_slots, last_token, table, x, buckets, mul_prev, mul_cur) -> None:
        T = x.shape[0]
        before = last_token.clone()
        for t in range(T):
            slot, pos = int(token_slots[t]), int(positions[t])
            row = buckets
            if slot >= 0 and pos > 0:
                inside = t > 0 and int(token_slots[t - 1]) == slot and int(positions[t - 1]) == pos - 1
                prev = int(tokens[t - 1]) if inside else int(before[slot])
                row = (prev * mul_prev + int(tokens[t]) * mul_cur) % buckets
            x[t] += table[row].float()
            if slot >= 0 and (t + 1 >= T or int(token_slots[t + 1]) != slot):
                last_token[slot] = int(tokens[t])

    def feed_tokens(self, dst, src, rows, n) -> None:
        dst[:n] = src[:n] if rows is None else src[rows[:n].long()]

    # ---- norm
    def norm(self, x, weight, bias, eps, out, rows=None, rms=False, pending=None) -> None:
        if pending is not None:  # what this stand-in leaves unfinished: a write into several residual streams, a gated sublayer
            self.finish(pending)
        src = x if rows is None else x[rows.long()]
        if rms:
            y = src / torch.sqrt((src * src).mean(-1, keepdim=True) + eps) * weight
            if bias is not None:
                y = y + bias
        else:
            y = F.layer_norm(src, (src.shape[-1],), weight, bias, eps)
        out.copy_(y.to(out.dtype))

    def finish(self, pending) -> None:
        if hasattr(pending, "post_weight"):
            self.group_norm_step(pending.out, groups=pending.groups, eps=pending.eps, pending=pending)
            return
        self.streams_step(pending.streams, y=pending.y, mix=pending.mix, w_out=pending.w_out, x_out=pending.out)  # a product is never left unfinished here

    # ---- several residual streams
    def streams_step(self, streams, *, x_init=None, y=None, mix=None, w_out=None, w_in=None, norm_weight=None, eps=0.0, h_out=None, x_out=None,
                     rows=None, defer_out=None, y_pending=None):
        assert y_pending is None, "this stand-in never leaves a product unfinished"
        if defer_out is not None:
            from types import SimpleNamespace

            return SimpleNamespace(out=defer_out, streams=streams, y=y, mix=mix, w_out=w_out, y_pending=None)
        xs = streams if x_init is None else x_init[None].expand(streams.shape[0], -1, -1)
        if y is not None:
            xs = torch.einsum("st,sid->tid", mix, xs) + w_out[:, None, None] * y[None]
        if rows is None and (y is not None or x_init is not None):
            streams.copy_(xs)
        u = xs.sum(0) if w_in is None else torch.einsum("s,sid->id", w_in, xs)
        if x_out is not None and rows is None:
            x_out.copy_(u)
        if h_out is not None:
            src = u if rows is None else u[rows.long()]
            h_out.copy_((src / torch.sqrt((src * src).mean(-1, keepdim=True) + eps) * norm_weight).to(h_out.dtype))
        return None

    # ---- rotation of pairs
    def rotary_pairs(self, q, k, head_dim, freqs, positions, magnitude=1.0) -> None:
        n = 2 * freqs.numel()
        a = positions.float()[:, None] * freqs[None, :]
        cos, sin = (torch.cos(a) * magnitude)[:, None, :], (torch.sin(a) * magnitude)[:, None, :]
        for t in (q, k):
            if t is None:
                continue
            x = t.float().reshape(t.shape[0], -1, head_dim).clone()
            u, v = x[..., 0:n:2].clone(), x[..., 1:n:2].clone()
            x[..., 0:n:2] = u * cos - v * sin
            x[..., 1:n:2] = v * cos + u * sin
            t.copy_(x.reshape(t.shape[0], -1).to(t.dtype))

    # ---- block-diagonal products
    BLOCK_LINEAR_MAX_ROWS = 128

    def block_linear(self, a, w, bias, out) -> None:
        B, n_out, n_in = w.shape
        y = torch.einsum("tbi,boi->tbo", a.float().view(a.shape[0], B, n_in), w.float()).reshape(a.shape[0], B * n_out)
        if bias is not None:
            y = y + bias
        out.copy_(y.to(out.dtype))

    # ---- the recurrent branch
    def causal_conv(self, x, taps, bias, state, token_slots, u) -> None:
        T, C = x.shape
        K = taps.shape[1]
        for t in range(T):
            slot = int(token_slots[t])
            if slot < 0:
                u[t] = 0
                continue
            n_back = 0
            while n_back < K - 1 and t - n_back - 1 >= 0 and int(token_slots[t - n_back - 1]) == slot:
                n_back += 1
            acc = bias.clone() if bias is not None else torch.zeros(C)
            for k in range(K):
                xv = x[t - k].float() if k <= n_back else state[slot, n_back + K - 1 - k]
                acc = acc + taps[:, K - 1 - k] * xv
            u[t] = acc.to(u.dtype)

    def gated_recurrence(self, u, gates, y, x, decay, state, token_slots, out, n_blocks, out_scale=1.0) -> None:
        T, C = u.shape
        K = state.shape[1]
        bw = C // n_blocks
        g = gates.view(T, n_blocks, 2, bw)
        t = 0
        while t < T:
            slot = int(token_slots[t])
            if slot < 0:
                out[t] = 0
                t += 1
                continue
            n = 1
            while t + n < T and int(token_slots[t + n]) == slot:
                n += 1
            S = state[slot, K - 1].clone()
            for i in range(n):
                r = torch.sigmoid(g[t + i, :, 0].reshape(C))
                ig = torch.sigmoid(g[t + i, :, 1].reshape(C))
                log_a = decay * r
                S = torch.exp(log_a) * S + torch.sqrt(-torch.expm1(2 * log_a)) * ig * u[t + i].float()
                out[t + i] = (S * F.gelu(y[t + i].float(), approximate="tanh") * out_scale).to(out.dtype)
            state[slot, K - 1] = S
            hist = torch.cat([state[slot, :K - 1], x[t:t + n].float()], 0)
            state[slot, :K - 1] = hist[hist.shape[0] - (K - 1):]
            t += n

    # ---- norms in groups around gated sublayers
    @staticmethod
    def _group_norm(v, w, groups, eps):
        T, D = v.shape
        parts = v.view(T, groups, D // groups)
        return (parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)).reshape(T, D) * w

    def group_norm_step(self, x, *, groups, eps, y=None, gate=None, post_weight=None, mult=1.0, weight=None, h_out=None, rows=None, defer=False,
                        pending=None, plain_read=False):
        if pending is not None:
            assert pending.out is x and y is None
            y, gate, post_weight, mult = pending.y, pending.gate, pending.post_weight, pending.mult
        if defer:
            from types import SimpleNamespace

            return SimpleNamespace(out=x, y=y, gate=gate, post_weight=post_weight, mult=float(mult), groups=int(groups), eps=float(eps))
        cur = x
        if y is not None:
            z = y if gate is None else y * torch.sigmoid(gate.float())
            cur = x + mult * self._group_norm(z, post_weight, groups, eps)
            if rows is None:
                x.copy_(cur)
        if h_out is not None:
            src = cur if rows is None else cur[rows.long()]
            h_out.copy_((src if plain_read else self._group_norm(src, weight, groups, eps)).to(h_out.dtype))
        return None

    # ---- rotation, rotate-half layout
    def rotary_half(self, x, n_heads, head_stride, offset, freqs, positions) -> None:
        n = freqs.numel()
        if n == 0:
            return
        a = positions.float()[:, None] * freqs[None, :]
        cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
        v = x[:, :n_heads * head_stride].view(x.shape[0], n_heads, head_stride)
        lo, hi = v[:, :, offset:offset + n].float().clone(), v[:, :, offset + n:offset + 2 * n].float().clone()
        v[:, :, offset:offset + n] = (lo * cos - hi * sin).to(x.dtype)
        v[:, :, offset + n:offset + 2 * n] = (hi * cos + lo * sin).to(x.dtype)

    # ---- generalized delta rule
    def delta_rule(self, r, k, v, a_pre, g, w_pre, norm_weight, state, token_slots, out, n_heads, head_dim, norm_eps, key_eps, sharpness, max_runs=None) -> None:
        T, H, d = r.shape[0], n_heads, head_dim
        nw = norm_weight.view(H, d)
        for t in range(T):
            slot = int(token_slots[t])
            if slot < 0:
                out[t] = 0
                continue
            kf, rf, vf = (z[t].float().view(H, d) for z in (k, r, v))
            u = kf / torch.sqrt((kf * kf).sum(-1, keepdim=True) + key_eps)
            w = torch.exp(-sharpness * torch.sigmoid(w_pre[t].float().view(H, d)))
            a = torch.sigmoid(a_pre[t].float().view(H, d))
            S = state[slot]
            uS = torch.einsum("hi,hij->hj", u, S)
            S = w[:, :, None] * S - (a * u)[:, :, None] * uS[:, None, :] + kf[:, :, None] * vf[:, None, :]
            state[slot] = S
            o = torch.einsum("hij,hi->hj", S, rf)
            o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + norm_eps) * nw * torch.sigmoid(g[t].float().view(H, d))
            out[t] = o.reshape(-1).to(out.dtype)

    # ---- gated linear attention
    def gated_linear_attention(self, q, k, v, g, z, norm_weight, state, token_slots, out, n_heads, key_dim, value_dim, tau, q_scale, norm_eps,
                               gate="silu", max_runs=None) -> None:
        T, H, dk, dv = q.shape[0], n_heads, key_dim, value_dim
        nw = norm_weight.view(H, dv)
        for t in range(T):
            slot = int(token_slots[t])
            if slot < 0:
                out[t] = 0
                continue
            qf, kf = (u[t].float().view(H, dk) for u in (q, k))
            vf, gf = (u[t].float().view(H, dv) for u in (v, g))
            a = torch.exp(-F.softplus(-z[t].float().view(H, dk)) / tau)
            S = a[:, :, None] * state[slot] + kf[:, :, None] * vf[:, None, :]
            state[slot] = S
            o = torch.einsum("hij,hi->hj", S, qf * q_scale)
            o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + norm_eps) * nw
            o = o * (gf * torch.sigmoid(gf) if gate == "silu" else torch.sigmoid(gf))
            out[t] = o.reshape(-1).to(out.dtype)

    # ---- row kernels of gated feed-forwards and of branches with norms of their own
    def glu_activate(self, z, out, activation, limit=0.0, up_shift=0.0) -> None:
        F_ = z.shape[1] // 2
        gt, up = z[:, :F_].float(), z[:, F_:].float()
        if limit > 0:
            gt, up = gt.clamp(max=limit), up.clamp(-limit, limit)
        out.copy_((_act(activation)(gt) * (up + up_shift)).to(out.dtype))

    def norm_sum2(self, a, b, weight_a, weight_b, scale_a, scale_b, eps, y) -> None:
        def n(v, w):
            return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w

        y.copy_(scale_a * n(a, weight_a) + scale_b * n(b, weight_b))

    # ---- mixture of experts
    def moe_route(self, z, correction, chosen, weights, *, n_groups=1, keep=1, group_top=2, renormalize=False, softmax=False) -> None:
        T, E = z.shape
        top = chosen.shape[1]
        s = torch.softmax(z.float(), -1) if softmax else torch.sigmoid(z.float())
        c = s if correction is None else s + correction
        per = E // n_groups
        for t in range(T):
            ct = c[t].clone()
            if n_groups > 1:
                scores = [sum(sorted(ct[g * per:(g + 1) * per].tolist(), reverse=True)[:group_top]) for g in range(n_groups)]
                order = sorted(range(n_groups), key=lambda g: (-scores[g], g))
                for g in order[keep:]:
                    ct[g * per:(g + 1) * per] = -math.inf
            order = sorted(range(E), key=lambda e: (-float(ct[e]), e))[:top]
            chosen[t] = torch.tensor(order, dtype=torch.int32)
            wt = s[t][order]
            weights[t] = wt / wt.sum() if renormalize else wt

    @staticmethod
    def moe_tile_rows(pairs, n_experts) -> int:
        return 64 if pairs >= 32 * n_experts else 16

    def moe_max_tiles(self, pairs, n_experts, tile_rows=16) -> int:
        return pairs // tile_rows + n_experts + 1

    def moe_sort(self, chosen, n_experts, sorted_pairs, pos_of, tiles, meta, tile_rows=16, n_real=None) -> None:
        flat = chosen.reshape(-1).long()
        order = torch.sort(flat, stable=True).indices
        P = flat.numel()
        sorted_pairs[:P] = order.to(torch.int32)
        pos_of[order] = torch.arange(P, dtype=torch.int32)
        tl = tiles.view(-1, 3)
        n, at = 0, 0
        for e in range(n_experts):
            count = int((flat == e).sum())
            for i in range(0, count if n_real is None or e < n_real else 0, tile_rows):
                tl[n] = torch.tensor([e, at + i, min(tile_rows, count - i)], dtype=torch.int32)
                n += 1
            at += count
        meta[0] = n

    def moe_linear(self, a, w, out, tiles, meta, sorted_pairs, *, top, gather, glu=False, activation="none", tile_rows=16, limit=0.0, up_shift=0.0) -> None:
        tl = tiles.view(-1, 3)
        F_ = out.shape[1]
        for i in range(int(meta[0])):
            e, first, n = (int(v) for v in tl[i])
            pos = torch.arange(first, first + n)
            src = (sorted_pairs[pos].long() // top) if gather else pos
            y = a[src].float() @ w[e].float().t()
            if glu:
                gt, up = y[:, :F_], y[:, F_:]
                if limit > 0:
                    gt, up = gt.clamp(max=limit), up.clamp(-limit, limit)
                y = _act(activation)(gt) * (up + up_shift)
            out[pos] = y.to(out.dtype)

    def moe_combine(self, expert_out, pos_of, weights, y, accumulate=False, chosen=None, n_real=0, identity_in=None) -> None:
        T, top = weights.shape
        acc = y.clone() if accumulate else torch.zeros_like(y)
        for c in range(top):
            term = expert_out[pos_of.view(T, top)[:, c].long()]
            if identity_in is not None:
                term = torch.where((chosen[:, c] >= n_real)[:, None], identity_in.float(), term)
            acc = acc + weights[:, c:c + 1] * term
        y.copy_(acc)

    # ---- linear
    def linear(self, a, w, bias, out, activation="none", residual=None, may_leave_pending=False) -> None:
        y = a.float() @ w.float().t()
        if bias is not None:
            y = y + bias
        y = _act(activation)(y)
        if residual is not None:
            y = y + residual
        out.copy_(y.to(out.dtype))

    # ---- cache layout helpers:  keys [page][kvh][hd/8][ps][8], values [page][kvh][hd][ps]
    @staticmethod
    def k_view(k_pages, kvh, hd, ps):
        return k_pages.view(-1, kvh, hd // 8, ps, 8)

    @staticmethod
    def v_view(v_pages, kvh, hd, ps):
        return v_pages.view(-1, kvh, hd, ps)

    def kv_write(self, k, v, k_pages, v_pages, dest, n_kv_heads, head_dim, page_size, value_dim=None) -> None:
        vd = head_dim if value_dim is None else value_dim
        kv_ = self.k_view(k_pages, n_kv_heads, head_dim, page_size)
        vv_ = self.v_view(v_pages, n_kv_heads, vd, page_size)
        for t in range(k.shape[0]):
            d = int(dest[t])
            if d < 0:
                continue
            page, off = d // page_size, d % page_size
            kv_[page, :, :, off, :] = k[t].view(n_kv_heads, head_dim // 8, 8)
            vv_[page, :, :, off] = v[t].view(n_kv_heads, vd)

    def gather_kv(self, k_pages, v_pages, table_row, lo, hi, n_kv_heads, head_dim, page_size, value_dim=None):
        """Keys and values of positions lo..hi-1 of one request: [kvh, n, hd] (values [kvh, n, value_dim])."""
        kv_ = self.k_view(k_pages, n_kv_heads, head_dim, page_size)
        vv_ = self.v_view(v_pages, n_kv_heads, head_dim if value_dim is None else value_dim, page_size)
        ks, vs = [], []
        for p in (lo if hi is None else range(lo, hi)):  # lo may be a list of positions
            page = int(table_row[p // page_size])
            assert page >= 0, "a key inside the window has no page"
            ks.append(kv_[page, :, :, p % page_size, :].reshape(n_kv_heads, head_dim))
            vs.append(vv_[page, :, :, p % page_size])
        return torch.stack(ks, 1), torch.stack(vs, 1)

    # ---- attention
    def paged_attention(self, q, out, k_pages, v_pages, meta, *, n_heads, n_kv_heads, head_dim, page_size, scale, window,
                        block_tables, k_new=None, v_new=None, dest=None, softcap=None, score_bias=None) -> bool:
        if k_new is not None:
            return False  # this stand-in never writes the cache inside attention: the caller calls kv_write
        T = q.shape[0]
        g = n_heads // n_kv_heads
        for t in range(T):
            pos = int(meta.positions[t])
            row = block_tables[int(meta.token_seq[t])]
            lo = max(0, pos - window + 1) if window else 0
            ks, vs = self.gather_kv(k_pages, v_pages, row, lo, pos + 1, n_kv_heads, head_dim, page_size)
            qt = q[t].float().view(n_heads, head_dim) * scale
            ks = ks.float().repeat_interleave(g, 0)  # [H, n, hd]
            vs = vs.float().repeat_interleave(g, 0)
            s = torch.einsum("hd,hnd->hn", qt, ks)
            if score_bias is not None:  # [heads, L]: entry min(distance, L - 1) of the head's row
                dist = (pos - torch.arange(lo, pos + 1)).clamp(max=score_bias.shape[1] - 1)
                s = s + score_bias.float().cpu()[:, dist]
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            p = torch.softmax(s, -1)
            if q.dtype == torch.bfloat16:
                p = p.to(torch.bfloat16).float()
            o = torch.einsum("hn,hnd->hd", p, vs)
            out[t] = o.reshape(-1).to(out.dtype)
        return False

    # ---- row-wise steps of layers that are not GPT-2's
    def head_prepare(self, qk, n_norm, head_dim, eps, v=None, v_first=None, n_blend=0, value_dim=0, blend=None, norm_dim=None,
                     norm_weight=None) -> None:
        if n_norm:
            x = qk[:, :n_norm * head_dim].float().view(qk.shape[0], n_norm, head_dim)
            x = x / torch.sqrt((x * x).sum(-1, keepdim=True) / (norm_dim or head_dim) + eps)
            if norm_weight is not None:
                x = x * norm_weight
            qk[:, :n_norm * head_dim] = x.reshape(qk.shape[0], -1).to(qk.dtype)
        if n_blend:
            lam = float(blend.reshape(-1)[0])
            v.copy_(((1.0 - lam) * v.float() + lam * v_first.float()).to(v.dtype))

    def head_prepare_write(self, q, k, v, k_pages, v_pages, dest, n_heads, n_kv_heads, head_dim, value_dim, page_size, eps, v_first=None,
                           blend=None, norm_dim=None, rotary_freqs=None, positions=None, q_norm_weight=None, k_norm_weight=None,
                           rotary_magnitude=1.0) -> None:
        k, v = k.clone(), v.clone()
        weighted = q_norm_weight is not None or k_norm_weight is not None
        if rotary_freqs is not None and not weighted:
            self.rotary_pairs(q, k, head_dim, rotary_freqs, positions, rotary_magnitude)
        if eps is not None:
            self.head_prepare(q, n_heads, head_dim, eps, norm_dim=norm_dim, norm_weight=q_norm_weight)
            self.head_prepare(k, n_kv_heads, head_dim, eps, norm_dim=norm_dim, norm_weight=k_norm_weight)
        if rotary_freqs is not None and weighted:  # a norm with a weight comes before the rotation
            self.rotary_pairs(q, k, head_dim, rotary_freqs, positions, rotary_magnitude)
        if v_first is not None:
            self.head_prepare(None, 0, 0, 0.0, v=v, v_first=v_first, n_blend=n_kv_heads, value_dim=value_dim, blend=blend)
        self.kv_write(k, v, k_pages, v_pages, dest, n_kv_heads, head_dim, page_size, value_dim=value_dim)

    def head_norm_rotate(self, q, k, n_heads, n_kv_heads, head_dim, eps, norm_dim=None, q_norm_weight=None, k_norm_weight=None, rotary_freqs=None,
                         positions=None, rotary_magnitude=1.0) -> None:
        if eps is not None:
            self.head_prepare(q, n_heads, head_dim, eps, norm_dim=norm_dim, norm_weight=q_norm_weight)
            self.head_prepare(k, n_kv_heads, head_dim, eps, norm_dim=norm_dim, norm_weight=k_norm_weight)
        if rotary_freqs is not None:
            self.rotary_pairs(q, k, head_dim, rotary_freqs, positions, rotary_magnitude)

    def norm_write_latent(self, c, weight, eps, norm_dim, k_pages, v_pages, dest, page_size) -> None:
        self.head_prepare(c, 1, c.shape[1], eps, norm_dim=norm_dim, norm_weight=weight)
        self.kv_write(c, c, k_pages, v_pages, dest, 1, c.shape[1], page_size)

    def latent_rope_write(self, kv, latent_dim, weight, eps, norm_dim, q, n_heads, q_head, q_offset, freqs, positions, k_pages, v_pages, dest,
                          page_size) -> None:
        KD = kv.shape[1]
        self.head_prepare(kv, 1, latent_dim, eps, norm_dim=norm_dim, norm_weight=weight)
        if freqs is not None and freqs.numel():
            self.rotary_half(kv, 1, KD, latent_dim, freqs, positions)
            if q is not None:
                self.rotary_half(q, n_heads, q_head, q_offset, freqs, positions)
        self.kv_write(kv, kv[:, :latent_dim], k_pages, v_pages, dest, 1, KD, page_size, value_dim=latent_dim)

    def recurrent_tokens(self, x, y, taps, conv_bias, gate_weight, gate_bias, decay, state, token_slots, out, out_scale=1.0) -> None:
        u = torch.empty_like(x)
        self.causal_conv(x, taps, conv_bias, state, token_slots, u)
        gates = torch.empty(x.shape[0], 2 * x.shape[1])
        self.block_linear(u, gate_weight, gate_bias, gates)
        self.gated_recurrence(u, gates, y, x, decay, state, token_slots, out, gate_weight.shape[0], out_scale)

    def poly_norm(self, z, coefficients, eps, out) -> None:
        u = z.float()
        c = [float(x) for x in coefficients]

        def n(w):
            return w / torch.sqrt((w * w).mean(-1, keepdim=True) + eps)

        out.copy_((c[0] * n(u) + c[1] * n(u * u) + c[2] * n(u * u * u) + c[3]).to(out.dtype))

    def head_talk(self, o, talk, gate, out, n_heads, n_kv_heads, value_dim, out_scale=1.0, gate_elements=False) -> None:
        T = out.shape[0]
        if talk is None:
            a = o.view(T, n_heads, value_dim)
        else:
            ov = o.view(T, n_heads, n_kv_heads, value_dim)
            own = torch.arange(n_heads) // (n_heads // n_kv_heads)
            a = torch.einsum("hg,tghd->thd", talk.float(), ov[:, :, own, :])  # [t, g, h, d]: weights of g on the values of h's own head
        if gate is not None:
            a = a * (torch.sigmoid(gate.float()).view(T, n_heads, value_dim) if gate_elements else torch.sigmoid(gate.float())[:, :, None])
        out.copy_((a * out_scale).reshape(T, -1).to(out.dtype))

    def stream_average(self, streams, x, weights, n, defer=False) -> None:
        streams[n - 1].copy_(x)
        acc = torch.zeros_like(x)
        for j in range(n):
            acc += weights[j] * streams[j]
        x.copy_(acc)

    def attention_values(self, q, out, k_pages, v_pages, meta, *, n_heads, n_kv_heads, head_dim, value_dim, all_value_heads, page_size,
                         scale, window, block_tables, softcap=None, slopes=None, chunk=None, sinks=None, keep_first=0) -> None:
        T = q.shape[0]
        g = n_heads // n_kv_heads
        o = out.view(T, n_heads, n_kv_heads if all_value_heads else 1, value_dim)
        for t in range(T):
            pos = int(meta.positions[t])
            row = block_tables[int(meta.token_seq[t])]
            lo = max(0, pos - window + 1) if window else 0
            if chunk:
                lo = max(lo, pos // chunk * chunk)
            seen = list(range(min(keep_first, lo))) + list(range(lo, pos + 1))  # the kept first positions, then the window
            ks, vs = self.gather_kv(k_pages, v_pages, row, seen, None, n_kv_heads, head_dim, page_size, value_dim)
            s = torch.einsum("hd,hnd->hn", q[t].float().view(n_heads, head_dim), ks.float().repeat_interleave(g, 0)) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            if slopes is not None:
                s = s - slopes.float()[:, None] * (pos - torch.tensor(seen)).float()[None, :]
            if sinks is not None:  # a score without a key and without a value in the denominator
                p = torch.softmax(torch.cat([s, sinks.float()[:, None]], -1), -1)[:, :-1]
            else:
                p = torch.softmax(s, -1)
            if all_value_heads:
                o[t] = torch.einsum("hn,cnd->hcd", p, vs.float())
            else:
                o[t, :, 0] = torch.einsum("hn,hnd->hd", p, vs.float().repeat_interleave(g, 0))

    # ---- sampling
    def sample(self, logits, temperatures, keys, positions, out_tokens, out_logprobs) -> None:
        for r in range(logits.shape[0]):
            lg = logits[r].float()
            temp = float(temperatures[r])
            if temp == 0.0:
                scaled = lg
                tok = int(torch.argmax(scaled))
            else:
                scaled = lg / temp
                noise = gumbel_noise(int(keys[r, 0]), int(keys[r, 1]), int(positions[r]), lg.shape[0])
                tok = int(torch.argmax(scaled + noise))
            out_tokens[r] = tok
            out_logprobs[r] = scaled[tok] - torch.logsumexp(scaled, -1)
