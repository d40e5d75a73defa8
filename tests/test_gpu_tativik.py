"""Tativik on the GPU: every kernel of its layers against the plain implementation's function of the same mechanism, then
whole models through the step function, ``bin/trace_run`` and the engine's own entry point, in 32-bit and bfloat16."""
import math
import os

import pytest
import torch

import plain_tativik as P
import traces as TR
from helpers import make_meta, random_block_tables
from tativik_configs import TAT

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def K():
    from levanter_amd.kernels import get_kernels

    return get_kernels()


def tol(dtype, f32=2e-5, bf16=2e-2):
    return dict(rtol=f32, atol=f32) if dtype == torch.float32 else dict(rtol=bf16, atol=bf16)


def bfn(x):
    """Numbers that bfloat16 holds exactly, as float64."""
    return x.to(torch.bfloat16).double()


def dev(x, dtype=torch.float32):
    return x.to(dtype).to(DEV)


# ------------------------------------------------------------------------------------------------ kernels
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,D,G", [(7, 64, 2), (33, 30, 5), (3, 257, 1), (2, 1000, 4), (1, 8, 8), (5, 4096, 2), (4, 600, 50)])
def test_group_norm_with_the_gated_write_of_the_sublayer_before(dtype, T, D, G):
    g = torch.Generator().manual_seed(D + G)
    x0, y = torch.randn(T, D, generator=g), torch.randn(T, D, generator=g) * 3
    gate = bfn(torch.randn(T, D + 8, generator=g))
    w, pw = 1 + 0.2 * torch.randn(D, generator=g), 1 + 0.2 * torch.randn(D, generator=g)
    eps, mult = 1e-5, 0.7
    kern = K()
    # the read by itself
    x = dev(x0)
    h = torch.empty(T, D, dtype=dtype, device=DEV)
    kern.group_norm_step(x, groups=G, eps=eps, weight=dev(w), h_out=h)
    torch.testing.assert_close(h.cpu().double(), P.group_rms_norm(x0.double(), w.double(), G, eps), **tol(dtype))
    assert torch.equal(x.cpu(), x0)
    # a pending write, done by the next read's pass; the gate comes as a slice of a wider product, in the compute dtype
    gd = dev(gate, dtype)[:, 8:]
    pending = kern.group_norm_step(x, groups=G, eps=eps, y=dev(y), gate=gd, post_weight=dev(pw), mult=mult, defer=True)
    assert pending is not None and torch.equal(x.cpu(), x0)  # nothing has run
    kern.group_norm_step(x, groups=G, eps=eps, weight=dev(w), h_out=h, pending=pending)
    x1 = x0.double() + mult * P.group_rms_norm(y.double() * torch.sigmoid(gate[:, 8:]), pw.double(), G, eps)
    torch.testing.assert_close(x.cpu().double(), x1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h.cpu().double(), P.group_rms_norm(x1, w.double(), G, eps), **tol(dtype))
    # the write by itself leaves the same bits
    again = dev(x0)
    kern.finish(kern.group_norm_step(again, groups=G, eps=eps, y=dev(y), gate=gd, post_weight=dev(pw), mult=mult, defer=True))
    assert torch.equal(again, x)
    # chosen rows (one named twice): write and norm of the selection, nothing is stored
    rows = torch.tensor([T - 1, 0, T - 1], dtype=torch.int32, device=DEV)
    pending = kern.group_norm_step(again, groups=G, eps=eps, y=dev(y), gate=None, post_weight=dev(pw), mult=-1.5, defer=True)
    before = again.clone()
    out = torch.empty(3, D, dtype=dtype, device=DEV)
    kern.group_norm_step(again, groups=G, eps=eps, weight=dev(w), h_out=out, rows=rows, pending=pending)
    x2 = x1 - 1.5 * P.group_rms_norm(y.double(), pw.double(), G, eps)
    torch.testing.assert_close(out.cpu().double(), P.group_rms_norm(x2, w.double(), G, eps)[rows.cpu().long()], **tol(dtype))
    assert torch.equal(again, before)
    # a 32-bit output (the embedding's norm)
    h32 = torch.empty(T, D, dtype=torch.float32, device=DEV)
    kern.group_norm_step(x, groups=G, eps=eps, weight=dev(w), h_out=h32)
    torch.testing.assert_close(h32.cpu().double(), P.group_rms_norm(x1, w.double(), G, eps), rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,stride,offset,dims", [(4, 24, 16, 8), (1, 48, 32, 16), (3, 18, 12, 4), (2, 64, 0, 64), (5, 40, 8, 0)])
def test_rotation_of_halves_in_place(dtype, H, stride, offset, dims):
    g = torch.Generator().manual_seed(stride)
    T = 9
    x = bfn(torch.randn(T, H * stride + 8, generator=g))
    positions = torch.tensor([0, 1, 2, 77, 1000, 4999, 3, 31, 640], dtype=torch.int32)
    base = 250.0
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64).float()
    xd = dev(x, dtype)
    K().rotary_half(xd, H, stride, offset, f.to(DEV), positions.to(DEV))
    want = x.clone()
    v = x[:, :H * stride].view(T, H, stride)
    want[:, :H * stride].view(T, H, stride)[:, :, offset:] = P.rotate_half(v[:, :, offset:], positions, dims, base)
    torch.testing.assert_close(xd.cpu().double(), want, **tol(dtype, f32=1.5e-3, bf16=2e-2))  # a 32-bit angle of 5,000 radians is good to 5e-4
    assert torch.equal(xd.cpu().double()[:, H * stride:], x[:, H * stride:])  # columns behind the heads stay


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,true_R,DR,dims,H,dk", [(32, 20, 16, 4, 3, 12), (16, 16, 16, 16, 1, 8), (64, 64, 48, 32, 5, 40), (48, 41, 8, 0, 2, 16), (224, 224, 32, 32, 16, 64)])
def test_rotation_norm_and_write_of_single_tokens_in_one_kernel_is_the_separate_kernels_bit_for_bit(dtype, R, true_R, DR, dims, H, dk):
    g = torch.Generator().manual_seed(R + DR)
    T, ps, n_pages = 7, 16, 12
    KD, qh = R + DR, dk + DR
    kv0 = torch.randn(T, KD + 16, generator=g)
    kv0[:, true_R:R] = 0
    q0 = torch.randn(T, H * qh, generator=g)
    w = torch.cat([1 + 0.2 * torch.randn(true_R, generator=g), torch.zeros(R - true_R)]).to(DEV)
    f = torch.tensor([77.0 ** (-2.0 * i / max(dims, 1)) for i in range(dims // 2)], dtype=torch.float32, device=DEV)
    positions = torch.tensor([0, 5, 130, 4000, 17, 1, 64], dtype=torch.int32, device=DEV)
    dest = torch.tensor([3 * ps + 1, 0, 11 * ps + 15, -1, 5 * ps + 7, 5 * ps + 8, 2 * ps], dtype=torch.int32, device=DEV)
    outs = []
    for fused in (True, False):
        kv, q = dev(kv0, dtype)[:, 8:8 + KD], dev(q0, dtype)
        kp = torch.zeros(n_pages, KD * ps, dtype=dtype, device=DEV)
        vp = torch.zeros(n_pages, R * ps, dtype=dtype, device=DEV)
        if fused:
            K().latent_rope_write(kv, R, w, 1e-5, true_R, q, H, qh, dk, f, positions, kp, vp, dest, ps)
        else:
            K().rotary_half(q, H, qh, dk, f, positions)
            K().rotary_half(kv, 1, KD, R, f, positions)
            K().head_prepare(kv[:, :R], 1, R, 1e-5, norm_dim=true_R, norm_weight=w)
            K().kv_write(kv, kv[:, :R], kp, vp, dest, 1, KD, ps, value_dim=R)
        outs.append((kv.clone(), q, kp, vp))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert outs[0][2].any() and outs[0][3].any()
    if dims:
        want = P.rotate_half(q0.to(dtype).double().view(T, H, qh)[:, :, dk:], positions.cpu(), dims, 77.0)
        torch.testing.assert_close(outs[0][1].cpu().double().view(T, H, qh)[:, :, dk:], want, **tol(dtype, f32=1e-3, bf16=2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Q,true_Q,heads", [(1024, 1024, 1), (520, 513, 2), (2048, 2000, 1)])
def test_rms_norm_with_a_weight_of_a_wide_head(dtype, Q, true_Q, heads):
    """A head of 512 elements and more takes a workgroup instead of a wave (the queries' latent of a wide model)."""
    g = torch.Generator().manual_seed(Q)
    buf = bfn(torch.randn(5, heads * Q + 16, generator=g))
    for h in range(heads):
        buf[:, h * Q + true_Q:(h + 1) * Q] = 0
    w = torch.cat([1 + 0.2 * torch.randn(true_Q, generator=g), torch.zeros(Q - true_Q)])
    b = dev(buf, dtype)
    K().head_prepare(b, heads, Q, 1e-5, norm_dim=true_Q, norm_weight=w.to(DEV))
    got = b.cpu().double()
    for h in range(heads):
        torch.testing.assert_close(got[:, h * Q:h * Q + true_Q], P.rms_norm(buf[:, h * Q:h * Q + true_Q], w[:true_Q].double(), 1e-5), **tol(dtype))
        assert not got[:, h * Q + true_Q:(h + 1) * Q].any()
    assert torch.equal(got[:, heads * Q:], buf[:, heads * Q:])


def delta_inputs(T, H, d, g, dtype):
    C = H * d
    stride = 5 * C + 8
    p = torch.randn(T, stride, generator=g)
    p[:, C:2 * C] *= 1.5
    p = bfn(p)
    w_pre = torch.randn(T, C, generator=g) * 2
    nw = 1 + 0.2 * torch.randn(C, generator=g)
    return p, w_pre, nw


def plain_delta(p, w_pre, nw, H, d, eps, state=None):
    T, C = p.shape[0], H * d
    r, k, v, a_pre, gt = (p[:, i * C:(i + 1) * C].view(T, H, d) for i in range(5))
    w = torch.exp(-P.DECAY_SHARPNESS * torch.sigmoid(w_pre.double().view(T, H, d)))
    o, S = P.delta_rule_scan(r, k, v, w, torch.sigmoid(a_pre), state)
    o = P.rms_norm(o, None, eps).reshape(T, C) * nw.double() * torch.sigmoid(gt.reshape(T, C))
    return o, S


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d", [(2, 16), (3, 10), (1, 64), (4, 48), (2, 128), (1, 1), (1, 200)])
@pytest.mark.parametrize("prompt_path", [False, True])
def test_the_delta_rule_carries_its_state_through_any_cutting(dtype, H, d, prompt_path):
    """Two requests and a token of nobody, cut into steps of several sizes down to one token: outputs and the slots' states are
    the plain scan's; the slots of others stay as they are."""
    g = torch.Generator().manual_seed(H * 100 + d)
    C = H * d
    eps = 1e-5
    lens = {0: 37, 2: 24}
    data = {s: delta_inputs(n, H, d, g, dtype) for s, n in lens.items()}
    want = {s: plain_delta(p, w, data[s][2], H, d, eps) for s, (p, w, _) in data.items()}
    nw = data[0][2]
    want[2] = plain_delta(data[2][0], data[2][1], nw, H, d, eps)
    state = torch.zeros(4, H, d, d, device=DEV)
    state[1] = 7.0
    state[3] = float("nan")
    at = {0: 0, 2: 0}
    got = {0: [], 2: []}
    for sizes in ([(0, 5), (2, 1)], [(2, 2), (0, 1)], [(0, 20), (-1, 1), (2, 13)], [(0, 1)], [(2, 1)], [(2, 6), (0, 10)], [(2, 1)]):
        rows, wrows, slots = [], [], []
        for s, n in sizes:
            if s < 0:
                rows.append(torch.zeros(n, 5 * C + 8, dtype=torch.float64))
                wrows.append(torch.zeros(n, C))
            else:
                rows.append(data[s][0][at[s]:at[s] + n])
                wrows.append(data[s][1][at[s]:at[s] + n])
            slots += [s] * n
        p = dev(torch.cat(rows), dtype)
        out = torch.full((p.shape[0], C), float("nan"), dtype=dtype, device=DEV)
        K().delta_rule(*(p[:, i * C:(i + 1) * C] for i in range(5)), dev(torch.cat(wrows)), dev(nw), state, torch.tensor(slots, dtype=torch.int32, device=DEV),
                       out, H, d, eps, P.UNIT_KEY_EPS, P.DECAY_SHARPNESS, max_runs=len(sizes) if prompt_path else None)
        t = 0
        for s, n in sizes:
            if s < 0:
                assert not out[t:t + n].any()
            else:
                got[s].append(out[t:t + n].cpu().double())
                at[s] += n
            t += n
    for s in lens:
        assert at[s] == lens[s]
        torch.testing.assert_close(torch.cat(got[s]), want[s][0], **tol(dtype, f32=2e-4, bf16=3e-2))
        torch.testing.assert_close(state[s].cpu().double(), want[s][1], rtol=2e-4, atol=2e-4)
    assert bool((state[1] == 7.0).all()) and bool(state[3].isnan().all())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d", [(2, 16), (3, 10), (2, 128), (1, 256)])
def test_the_prompt_path_of_the_delta_rule_on_long_runs_beside_single_tokens(dtype, H, d):
    """Runs of 300 and 150 tokens, two single tokens and a token of nobody in one step, from states that are not zero."""
    g = torch.Generator().manual_seed(d)
    C = H * d
    lens = [(0, 300), (3, 1), (-1, 1), (1, 150), (2, 1)]
    state0 = torch.randn(4, H, d, d, generator=g) * 0.3
    state = state0.to(DEV)
    rows, wrows, slots, want = [], [], [], []
    nw = 1 + 0.2 * torch.randn(C, generator=g)
    for s, n in lens:
        p, w_pre, _ = delta_inputs(n, H, d, g, dtype)
        rows.append(p)
        wrows.append(w_pre)
        slots += [s] * n
        want.append(plain_delta(p, w_pre, nw, H, d, 1e-5, state0[s].double()) if s >= 0 else (torch.zeros(n, C, dtype=torch.float64), None))
    p = dev(torch.cat(rows), dtype)
    out = torch.full((p.shape[0], C), float("nan"), dtype=dtype, device=DEV)
    K().delta_rule(*(p[:, i * C:(i + 1) * C] for i in range(5)), dev(torch.cat(wrows)), dev(nw), state, torch.tensor(slots, dtype=torch.int32, device=DEV), out,
                   H, d, 1e-5, P.UNIT_KEY_EPS, P.DECAY_SHARPNESS, max_runs=7)
    torch.testing.assert_close(out.cpu().double(), torch.cat([w[0] for w in want]), **tol(dtype, f32=5e-4, bf16=3e-2))
    for (s, n), w in zip(lens, want):
        if s >= 0:
            torch.testing.assert_close(state[s].cpu().double(), w[1], rtol=5e-4, atol=5e-4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_of_the_delta_rule_keeps_its_digits(dtype):
    """400 single tokens with weak decay and strong removal along keys that repeat: the state neither drifts nor blows up."""
    H, d, T = 2, 32, 400
    g = torch.Generator().manual_seed(5)
    p, w_pre, nw = delta_inputs(T, H, d, g, dtype)
    C = H * d
    p[:, C:2 * C] = p[:8, C:2 * C].repeat(T // 8, 1)  # eight keys in turn
    w_pre[:] = -6.0  # decay of nearly one
    p[:, 3 * C:4 * C] = 6.0  # removal rate of nearly one
    want, S = plain_delta(p, w_pre, nw, H, d, 1e-5)
    state = torch.zeros(1, H, d, d, device=DEV)
    outs = []
    for t in range(T):
        row = dev(p[t:t + 1], dtype)
        out = torch.empty(1, C, dtype=dtype, device=DEV)
        K().delta_rule(*(row[:, i * C:(i + 1) * C] for i in range(5)), dev(w_pre[t:t + 1]), dev(nw), state, torch.zeros(1, dtype=torch.int32, device=DEV), out,
                       H, d, 1e-5, P.UNIT_KEY_EPS, P.DECAY_SHARPNESS)
        outs.append(out.cpu().double())
    torch.testing.assert_close(torch.cat(outs), want, **tol(dtype, f32=5e-4, bf16=3e-2))
    torch.testing.assert_close(state[0].cpu().double(), S, rtol=5e-4, atol=5e-4)


@pytest.mark.parametrize("T,E,G,keep,top", [(37, 8, 4, 2, 2), (5, 16, 4, 3, 2), (64, 12, 1, 1, 3), (3, 6, 6, 2, 2), (200, 64, 8, 4, 6), (9, 2, 1, 1, 1),
                                             (11, 9, 3, 1, 3), (4, 256, 8, 4, 8)])
def test_the_router(T, E, G, keep, top):
    g = torch.Generator().manual_seed(E * 10 + top)
    z = torch.randn(T, E, generator=g) * 1.5
    corr = torch.randn(E, generator=g) * 0.5 - (1.0 if E == 6 else 0.0)  # E == 6: every choice score is negative
    chosen = torch.empty(T, top, dtype=torch.int32, device=DEV)
    weights = torch.empty(T, top, dtype=torch.float32, device=DEV)
    K().moe_route(dev(z), dev(corr), chosen, weights, n_groups=G, keep=keep, group_top=2)
    wc, ww = P.route(z.double(), corr.double(), top, G, keep)
    s = torch.sigmoid(z.double())
    for t in range(T):
        assert sorted(chosen[t].tolist()) == sorted(wc[t].tolist()), f"token {t}"
        torch.testing.assert_close(weights[t].cpu().double(), s[t][chosen[t].cpu().long()], rtol=1e-5, atol=1e-6)
    ties = torch.full((2, E), 0.3)  # all scores equal: the groups and the experts with the lower index win
    K().moe_route(dev(ties), None, chosen[:2], weights[:2], n_groups=G, keep=keep, group_top=2)
    assert chosen[0].tolist() == chosen[1].tolist() == list(range(top)) if top <= keep * (E // G) else True
    K().moe_route(dev(z), None, chosen, weights, n_groups=1, keep=1, renormalize=True)  # no correction, no groups, weights that sum to one
    assert sorted(chosen[1].tolist()) == sorted(z[1].topk(top).indices.tolist())
    torch.testing.assert_close(weights.sum(-1).cpu(), torch.ones(T), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,D,F,E,top", [(37, 64, 24, 8, 2), (1, 32, 8, 2, 1), (300, 96, 48, 12, 3), (5, 40, 13, 5, 2), (64, 256, 96, 4, 4), (9, 128, 200, 3, 1), (700, 64, 24, 40, 2)])
@pytest.mark.parametrize("rows", [16, 64])
def test_the_experts_products_over_tokens_sorted_by_expert(dtype, T, D, F, E, top, rows):
    g = torch.Generator().manual_seed(T + F)
    h = bfn(torch.randn(T, D, generator=g))
    W = {}
    for e in range(E):
        W[f"m.e{e}.gate"] = bfn(torch.randn(F, D, generator=g) / math.sqrt(D))
        W[f"m.e{e}.up"] = bfn(torch.randn(F, D, generator=g) / math.sqrt(D))
        W[f"m.e{e}.down"] = bfn(torch.randn(D, F, generator=g) / math.sqrt(F))
    chosen = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if T > 20:
        chosen[:18, 0] = 1  # more rows for one expert than a tile holds
        chosen[:18, 1:] = torch.tensor([e for e in range(E) if e != 1][:top - 1], dtype=torch.int32)
    weights = torch.rand(T, top, generator=g)
    Fp = (F + 7) // 8 * 8
    w_in = torch.zeros(E, 2 * Fp, D, dtype=torch.float64)
    w_down = torch.zeros(E, D, Fp, dtype=torch.float64)
    for e in range(E):
        w_in[e, :F], w_in[e, Fp:Fp + F], w_down[e, :, :F] = W[f"m.e{e}.gate"], W[f"m.e{e}.up"], W[f"m.e{e}.down"]
    kern = K()
    Pn = T * top
    tables = torch.full((2 * Pn + 3 * kern.moe_max_tiles(Pn, E, rows) + 1,), -7, dtype=torch.int32, device=DEV)
    sorted_pairs, pos_of, meta, tiles = tables[:Pn], tables[Pn:2 * Pn], tables[2 * Pn:2 * Pn + 1], tables[2 * Pn + 1:]
    kern.moe_sort(chosen.to(DEV), E, sorted_pairs, pos_of, tiles, meta, tile_rows=rows)
    sp, po = sorted_pairs.cpu().long(), pos_of.cpu().long()
    assert sorted(sp.tolist()) == list(range(Pn)) and torch.equal(sp[po], torch.arange(Pn))
    flat = chosen.reshape(-1).long()
    assert torch.equal(flat[sp], flat[sp].sort().values)  # pairs of one expert lie together, experts in rising order
    n_tiles = int(meta[0])
    tl = tiles.cpu().view(-1, 3)[:n_tiles]
    covered = torch.cat([torch.arange(int(f), int(f) + int(n)) for _, f, n in tl])
    assert torch.equal(covered, torch.arange(Pn)) and all(bool((flat[sp][int(f):int(f) + int(n)] == int(e)).all()) and 0 < int(n) <= rows for e, f, n in tl)
    inner = torch.full((Pn, Fp), float("nan"), dtype=dtype, device=DEV)
    kern.moe_linear(dev(h, dtype), dev(w_in, dtype), inner, tiles, meta, sorted_pairs, top=top, gather=True, glu=True, activation="silu", tile_rows=rows)
    eo = torch.full((Pn, D), float("nan"), dtype=torch.float32, device=DEV)
    kern.moe_linear(inner, dev(w_down, dtype), eo, tiles, meta, sorted_pairs, top=top, gather=False, tile_rows=rows)
    y = torch.full((T, D), float("nan"), dtype=torch.float32, device=DEV)
    kern.moe_combine(eo, pos_of, dev(weights), y)
    want = torch.zeros(T, D, dtype=torch.float64)
    for t in range(T):
        for c in range(top):
            want[t] += weights[t, c].double() * P.expert(h[t:t + 1], W, f"m.e{int(chosen[t, c])}")[0]
    torch.testing.assert_close(y.cpu().double(), want, **tol(dtype, f32=5e-5, bf16=3e-2))
    base = torch.randn(T, D, generator=g)
    y2 = dev(base)
    kern.moe_combine(eo, pos_of, dev(weights), y2, accumulate=True)
    torch.testing.assert_close(y2.cpu().double(), base.double() + want, **tol(dtype, f32=5e-5, bf16=3e-2))


# ---- attention with a window and a sink over [latent | rotated key part] keys ---------------------------------------------------
def run_attention(dtype, H, dk, dv, runs, window, scale, q, k, v, sinks, ps=16, seed=0):
    """One key/value head that all query heads share, keys of dk and values of dv, as the latent attention stores them."""
    kern = K()
    kv_lens = [kv for _, kv in runs]
    n_pages = sum((n + ps - 1) // ps for n in kv_lens) + 3
    bt = random_block_tables(kv_lens, ps, n_pages, seed, DEV)
    k_pages = torch.full((n_pages, dk * ps), float("nan"), dtype=dtype, device=DEV)  # what a recycled page may hold
    v_pages = torch.full((n_pages, dv * ps), float("nan"), dtype=dtype, device=DEV)
    for s, n in enumerate(kv_lens):
        dest = torch.tensor([int(bt[s, p // ps]) * ps + p % ps for p in range(n)], dtype=torch.int32, device=DEV)
        kern.kv_write(dev(k[s], dtype), dev(v[s], dtype), k_pages, v_pages, dest, 1, dk, ps, value_dim=dv)
    meta = make_meta(runs, DEV)
    qq = dev(torch.cat(q), dtype)
    o = torch.empty(qq.shape[0], H, 1, dv, dtype=torch.float32, device=DEV)
    kern.attention_values(qq, o, k_pages, v_pages, meta, n_heads=H, n_kv_heads=1, head_dim=dk, value_dim=dv, all_value_heads=False,
                          page_size=ps, scale=scale, window=window, block_tables=bt, sinks=None if sinks is None else dev(sinks))
    return o.view(qq.shape[0], H * dv).cpu().double()


def plain_attention(H, dk, dv, runs, window, scale, q, k, v, sinks):
    outs = []
    for s, (q_len, kv_len) in enumerate(runs):
        full_q = torch.zeros(kv_len, H, dk, dtype=torch.float64)
        full_q[kv_len - q_len:] = q[s].view(q_len, H, dk)
        scores = torch.einsum("ihd,jd->hij", full_q, k[s]) * scale
        w = P.softmax_with_sink(scores, P.window_visible(kv_len, window), None if sinks is None else sinks.double())
        outs.append(torch.einsum("hij,jd->ihd", w, v[s])[kv_len - q_len:].reshape(q_len, H * dv))
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk,dv,window,sink", [(4, 32, 24, 24, True), (8, 48, 32, 16, True), (3, 64, 48, 70, False), (6, 24, 16, 5, True), (2, 256, 224, 200, True),
                                                 (34, 32, 16, 21, True), (5, 80, 64, None, True), (3, 16, 16, 1, True)])
def test_windowed_attention_with_sinks_prompts_portions_and_single_tokens(dtype, H, dk, dv, window, sink):
    g = torch.Generator().manual_seed(H * 100 + dk)
    runs = [(70, 70), (1, 130), (19, 83), (1, 1), (2, 2), (1, 17), (130, 261), (1, 48), (1, 241), (5, 245)]  # (queries, keys after the step)
    q = [bfn(torch.randn(ql, H * dk, generator=g)) for ql, _ in runs]
    k = [bfn(torch.randn(kl, dk, generator=g)) for _, kl in runs]
    v = [bfn(torch.randn(kl, dv, generator=g)) for _, kl in runs]
    sinks = bfn(torch.randn(H, generator=g) * 2) if sink else None
    scale = 2.0 / math.sqrt(dk)
    got = run_attention(dtype, H, dk, dv, runs, window, scale, q, k, v, sinks, seed=dk)
    want = plain_attention(H, dk, dv, runs, window, scale, q, k, v, sinks)
    torch.testing.assert_close(got, want, **tol(dtype, f32=3e-5, bf16=3e-2))
    if sink:  # the sink does matter: without it the weights are others
        assert (plain_attention(H, dk, dv, runs, window, scale, q, k, v, None) - want).abs().max() > 0.05


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("single", [True, False])
@pytest.mark.parametrize("window,ps", [(24, 16), (16, 16), (33, 16), (64, 32), (100, 16), (129, 64), (1, 16)])
def test_a_key_just_inside_and_just_outside_the_window(dtype, single, window, ps):
    """One key carries a value far from all others and a score that stands out. As the oldest key of the query's window it is the
    query's output (less the sink's share); one position older it must not be seen at all. The query is the last token of a
    prompt portion, or a single token; sequences shorter and longer than the window; a sink so large that it takes nearly all
    of one head's weight."""
    H, dk, dv = 4, 32, 16
    g = torch.Generator().manual_seed(window)
    sinks = torch.tensor([0.0, -1.0, 30.0, 1.0])
    for n in sorted({window, window + 1, 3 * window + 2, 2 * ps + 1}):
        for j, seen in ((n - window, True), (n - window - 1, False)):
            if j < 0:
                continue
            kk = bfn(torch.randn(n, dk, generator=g) * 0.05)
            qq = bfn(torch.randn(n, H, dk, generator=g))
            vv = bfn(torch.randn(n, dv, generator=g) * 0.1)
            kk[j] = qq[n - 1, H - 1]  # the last head's query finds its own direction there: a score of about dk
            vv[j] = 100.0
            ql = 1 if single else min(n, 37)
            runs = [(ql, n)]
            args = (H, dk, dv, runs, window, 1.0, [qq[n - ql:].reshape(ql, -1)], [kk], [vv], sinks)
            got = run_attention(dtype, *args, ps=ps, seed=n)
            want = plain_attention(*args)
            torch.testing.assert_close(got, want, **tol(dtype, f32=3e-5, bf16=3e-2))
            last = got[-1].view(H, dv)
            assert bool((last[H - 1] > 90).all()) == seen and (seen or bool((last[H - 1].abs() < 5).all())), f"key {j}, query {n - 1}, window {window}"
            assert bool((last[2].abs() < 1e-3).all()) or (seen and window == 1)  # the head whose sink is huge gives next to nothing


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_among_hundreds_through_the_latent_with_a_rotated_part(dtype):
    """The latent attention's kernels in the engine's order through the part itself, on its own: one far token among 900 is made
    to carry the rotated key part that the last query's first head looks for at that distance."""
    from levanter_amd.parts import BuildEnv, CacheUnitView, GroupView, StepContext
    from levanter_amd.parts.latent_attention import LatentAttention
    from levanter_amd.parts.spec import PartSpec

    H, dk, dr, dv, R, Q, D = 4, 16, 16, 8, 32, 24, 48
    n, far = 900, 3
    g = torch.Generator().manual_seed(2)
    m = {"heads": H, "dim": dk, "rot_dim": dr, "vdim": dv, "kv_rank": R, "q_rank": Q, "scale": 0.5, "rot": {"dims": dr, "base": 10000.0}}
    W = {"x.dq": bfn(torch.randn(Q, D, generator=g) / math.sqrt(D)), "x.dq.norm": bfn(1 + 0.2 * torch.randn(Q, generator=g)),
         "x.uq": bfn(torch.randn(H * (dk + dr), Q, generator=g) / math.sqrt(Q)), "x.dkv": bfn(torch.randn(R + dr, D, generator=g) / math.sqrt(D)),
         "x.dkv.norm": bfn(1 + 0.2 * torch.randn(R, generator=g)), "x.uk": bfn(torch.randn(H * dk, R, generator=g) / math.sqrt(R)),
         "x.uv": bfn(torch.randn(H * dv, R, generator=g) / math.sqrt(R)), "x.sink": bfn(torch.randn(H, generator=g)),
         "x.g": bfn(torch.randn(H, D, generator=g) / math.sqrt(D)), "x.o": bfn(torch.eye(D, H * dv))}
    h = bfn(torch.randn(n, D, generator=g))
    # the far token's rotated key part: the last query's (head 0) rotated part turned back by the distance, so that after both
    # rotations the two are parallel; its input is the least-squares solution for those rows of W_dkv
    cq = P.rms_norm(h[n - 1:] @ W["x.dq"].T, W["x.dq.norm"], 1e-5)
    q_rot = (cq @ W["x.uq"].T).view(H, dk + dr)[0, dk:]
    target = P.rotate_half(P.rotate_half(q_rot[None], torch.tensor([n - 1]), dr, 10000.0), torch.tensor([-far]), dr, 10000.0)[0]
    full = torch.cat([torch.zeros(R, dtype=torch.float64), target * 4])
    h[far] = bfn(torch.linalg.lstsq(W["x.dkv"], full[:, None]).solution[:, 0])
    want, _ = P.latent_attention(h, W, "x", m, 1e-5)
    h2 = h.clone()
    h2[far] = h[far + 1]
    assert (P.latent_attention(h2, W, "x", m, 1e-5)[0][-1] - want[-1]).abs().max() > 0.05  # the far token does stand out
    env = BuildEnv(dtype, torch.device(DEV), K())
    tensors = {"q_down.weight": W["x.dq"], "q_norm.weight": W["x.dq.norm"], "q.weight": W["x.uq"], "down.weight": W["x.dkv"],
               "latent_norm.weight": W["x.dkv.norm"], "up_k.weight": W["x.uk"], "up_v.weight": W["x.uv"], "sinks": W["x.sink"],
               "gate.weight": W["x.g"], "out.weight": W["x.o"]}
    part = LatentAttention(PartSpec("latent_attention", {"dim": D, "n_heads": H, "head_dim": dk, "value_dim": dv, "latent_dim": R, "query_latent_dim": Q,
                                                         "rope_dim": dr, "rotary": {"dims": dr, "base": 10000.0}, "scale": 0.5, "norm_eps": 1e-5,
                                                         "window": None, "sinks": True, "gate": True}), tensors, env)
    ps = 16
    req = part.cache_requirement()
    bt = random_block_tables([n], ps, 60, 1, DEV)
    kp = torch.full((60, req.head_dim * ps), float("nan"), dtype=dtype, device=DEV)
    vp = torch.full((60, req.v_dim * ps), float("nan"), dtype=dtype, device=DEV)
    got, at = [], 0
    for ql in (700, 199, 1):  # a long portion, a second one, a single token
        meta = make_meta([(ql, at + ql)], DEV)
        dest = torch.tensor([int(bt[0, t // ps]) * ps + t % ps for t in range(at, at + ql)], dtype=torch.int32, device=DEV)
        ctx = StepContext(kernels=K(), dtype=dtype, device=torch.device(DEV), n_tokens=ql, tokens=torch.zeros(ql, dtype=torch.int32, device=DEV),
                          attention=meta, seq_slots=torch.zeros(1, dtype=torch.int32, device=DEV), host={})
        unit = CacheUnitView(k_pages=kp, v_pages=vp, group=GroupView(ps, bt, dest))
        y = torch.empty(ql, D, dtype=torch.float32, device=DEV)
        part.compute(dev(h[at:at + ql], dtype), y, ctx, unit, True)
        ctx.settle()
        got.append(y.cpu().double())
        at += ql
    torch.testing.assert_close(torch.cat(got), want, **tol(dtype, f32=1e-4, bf16=5e-2))


# ------------------------------------------------------------------------------------------------ whole models
def model_folder(name, tmp, store):
    """bfloat16 folders get routers that decide by a wide margin: a choice by less than the inputs' rounding could fall either
    way there, and what follows would be another model's. Routers whose choice hangs on the input run in 32-bit."""
    raw, seed = TAT[name]
    W = P.random_weights(raw, seed, clear_routing=store == torch.bfloat16)
    return raw, W, P.write_folder(raw, W, os.path.join(str(tmp), name), store)


def row_error(got, want):
    """Difference of two rows of logits, mean taken off, relative to the spread of the wanted row."""
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / want.std(-1)).max().item()


LENGTHS = {"A": [70, 45, 100, 37, 64, 33], "B": [90, 130, 41, 200, 64, 17], "C": [40, 12, 30, 3], "D": [66, 21, 80, 5, 97]}


@pytest.mark.parametrize("name", list(TAT))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_all_cuttings(name, dtype, tmp_path):
    """Whole prompts, the last 32 tokens one by one, portions down to two tokens, and twice mixed with other requests in a pool
    of exactly the peak need (pages and slots are used again), through ``bin/trace_run``."""
    from test_gpu_replay import read_step, run_trace

    raw, W, d = model_folder(name, tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    reqs = TR.random_requests(raw["vocab"], LENGTHS[name], 21)
    plain = {rid: P.plain_logits(W, raw, t) for rid, t in reqs.items()}
    steps = TR.number(TR.trace_whole(reqs) + TR.trace_prefill_then_singles(reqs) + TR.trace_portions(reqs)
                      + TR.trace_mixed(reqs, seed=3) + TR.trace_mixed(reqs, seed=4, prefix="n"))
    out = run_trace(d, dtype, steps, TR.peak_tokens(steps), extra=("--max-seqs", "4"))
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    # every row ahead of a request's first close call of a router is held to the limit (the folder's routers are drawn so that
    # there is none in bfloat16; 32-bit rounding is far below any margin that occurs)
    safe = {rid: len(t) if dtype == "float32" else P.first_close_call(W, raw, t, 0.02) for rid, t in reqs.items()}
    assert all(safe[rid] == len(t) for rid, t in reqs.items())
    # bfloat16: every sublayer's result is normed again, so its rounding reaches the stream undamped; and a few positions are
    # ill-conditioned by the design itself (a first token whose key is nearly orthogonal to its receptance: the head norm of the
    # delta rule then divides a sum that cancels by its own size): one row in a hundred may miss the limit there
    limit = 1e-4 if dtype == "float32" else 1e-1
    worst, strict, loose, loose_ok, over = 0.0, 0, 0, 0, []
    at = {}
    for s in steps:
        k = s["step"]
        assert (k in want) == os.path.exists(os.path.join(out, f"{k}.f32"))
        got = read_step(out, k, raw["vocab"]).double() if k in want else None
        row = 0
        for e in s["entries"]:
            start = at.get(e["id"], 0)
            at[e["id"]] = start + len(e["tokens"])
            for w in e["want"]:
                err = row_error(got[row:row + 1], want[k][row:row + 1])
                if start + w < safe[e["id"][1:]]:
                    strict += 1
                    if err >= limit:
                        over.append(f"step {k} {e['id']} position {start + w}: {err}")
                    else:
                        worst = max(worst, err)
                else:
                    loose += 1
                    loose_ok += err < limit
                row += 1
        for rid in s["end"]:
            at.pop(rid, None)
    print(f"tativik {name} {dtype}: worst relative row error {worst:.3e} over {strict} rows; {loose_ok} of {loose} rows behind a close call within the limit")
    assert strict >= 100 and loose == 0
    assert len(over) <= (0 if dtype == "float32" else strict // 100), over[:10]


def _engine(d, dtype, **kw):
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import InferenceEngine

    cfg = InferenceEngineConfig(**{**dict(max_seqs=4, page_size=16, max_pages_per_seq=32, compute_dtype=dtype), **kw})
    return InferenceEngine.from_pretrained(d, cfg)


def check_greedy(W, raw, prompt, generated, margin, route_delta=0.0):
    logits = P.plain_logits(W, raw, list(prompt) + list(generated))
    clear = 0
    safe = P.first_close_call(W, raw, list(prompt) + list(generated), route_delta) if route_delta else len(prompt) + len(generated)
    for i, tok in enumerate(generated):
        if len(prompt) - 1 + i >= safe:  # from here on a router's close call may have gone the other way
            break
        row = logits[len(prompt) - 1 + i]
        top = row.topk(2).values
        if float(top[0] - top[1]) > margin:
            clear += 1
            assert int(row.argmax()) == tok, f"generated token {i}"
    return clear


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(dtype, tmp_path):
    from levanter_amd.engine import Request

    raw, W, d = model_folder("A", tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, raw["vocab"], (n,), generator=g).tolist() for n in (5, 17, 33, 1)]
    engine = _engine(d, dtype)
    res = engine.generate([Request(prompt_tokens=p, request_id=i, max_new_tokens=20) for i, p in enumerate(prompts)])
    assert [len(t) for t in res.tokens] == [20] * 4 and res.finish_reasons == ["length"] * 4
    margin = 1e-3 if dtype == "float32" else 0.2
    clear = sum(check_greedy(W, raw, p, out, margin, 0.0 if dtype == "float32" else 0.02) for p, out in zip(prompts, res.tokens))
    print(f"greedy {dtype}: {clear} of 80 positions decided by more than {margin}")
    assert clear >= (76 if dtype == "float32" else 30)
    engine.cache.check_invariants()
    assert engine.cache.n_free_slots == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_every_window_in_replayed_steps(dtype, tmp_path):
    """One prompt token, then 300 decoded ones: the windows (9, 24 and 37) pass over decoded tokens only, their group gives pages
    back on the way, the delta rule runs 300 steps from its slot, and from the third step on the steps are replayed from a
    graph. Then the first tokens of sequences of one, two and three tokens in one batch, in slots that were used before."""
    from levanter_amd.engine import Request

    raw, W, d = model_folder("A", tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    engine = _engine(d, dtype, max_pages=40)
    assert engine.model.graph_safe
    res = engine.generate([Request(prompt_tokens=[7], request_id=0, max_new_tokens=300)])
    out = res.tokens[0]
    assert len(out) == 300
    delta = 0.0 if dtype == "float32" else 0.02
    clear = check_greedy(W, raw, [7], out, 1e-3 if dtype == "float32" else 0.2, delta)
    print(f"long decoding {dtype}: {clear} of 300 positions decided clearly")
    assert clear >= (280 if dtype == "float32" else 100)
    res = engine.generate([Request(prompt_tokens=p, request_id=i + 1, max_new_tokens=3) for i, p in enumerate(([5], [9, 4], [1, 2, 3]))])
    for p, o in zip(([5], [9, 4], [1, 2, 3]), res.tokens):
        check_greedy(W, raw, p, o, 1e-3 if dtype == "float32" else 0.2, delta)
    engine.cache.check_invariants()


def test_the_command_line_generates_from_a_folder(tmp_path):
    """``python -m levanter_amd.main.sample_lm`` on a Tativik folder: greedy tokens are the plain implementation's."""
    import json
    import re
    import subprocess
    import sys

    raw, W, d = model_folder("D", tmp_path, torch.float32)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompts = [[3, 14, 15, 9, 2], [6]]
    p = subprocess.run([sys.executable, "-m", "levanter_amd.main.sample_lm", "--hf_checkpoint", d, "--prompt_ids", json.dumps(prompts),
                        "--temperature", "0", "--max_new_tokens", "12", "--n_rounds", "1", "--engine.compute_dtype", "float32",
                        "--engine.max_seqs", "2", "--engine.max_pages_per_seq", "4"], capture_output=True, text=True, cwd=root, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    found = re.findall(r"round 0 sequence (\d+) \(12 tokens, length\): (\[.*\])", p.stdout)
    assert len(found) == 2
    for i, toks in found:
        check_greedy(W, raw, prompts[int(i)], json.loads(toks), 1e-3)
