"""Tativik through the framework's step function, cache manager and parts on the CPU with the emulated kernels, against the
plain implementation: what differs here is a fault of the host logic (tables, pages, state slots, a layer that reads another
layer's cache unit, what sublayers hand each other within a step), not of a kernel. Also the plain implementation's own
mechanisms against direct statements of what they must do."""
import copy
import math
import os

import pytest
import torch

import plain_tativik as P
import traces as TR
from emulated_kernels import EmulatedKernels
from levanter_amd.cache import PagedKv, SlotState
from levanter_amd.config import ConfigError, InferenceEngineConfig, LmConfig, TativikConfig
from levanter_amd.engine import ModelRunner, StepEntry
from levanter_amd.engine.loading import load_model, make_cache
from levanter_amd.parts import BuildEnv
from levanter_amd.weights import WeightsError
from tativik_configs import TAT


def build(name, tmp, dtype=torch.float32):
    raw, seed = TAT[name]
    W = P.random_weights(raw, seed)
    d = P.write_folder(raw, W, os.path.join(str(tmp), name), torch.float32)
    env = BuildEnv(dtype, torch.device("cpu"), EmulatedKernels())
    config, model = load_model(d, env)
    return raw, W, model, env, config


LENGTHS = {"A": [70, 45, 100, 37, 64, 33], "B": [90, 130, 41, 17, 64], "C": [40, 12, 30], "D": [66, 21, 80, 5]}


@pytest.fixture(scope="module", params=list(TAT))
def setup(request, tmp_path_factory):
    raw, W, model, env, _ = build(request.param, tmp_path_factory.mktemp("tat"))
    reqs = TR.random_requests(raw["vocab"], LENGTHS[request.param], 5)
    plain = {rid: P.plain_logits(W, raw, t) for rid, t in reqs.items()}
    return raw, W, model, env, reqs, plain


def replay(model, env, steps, max_tokens, ps=16, max_seqs=4, after_step=None):
    cfg = InferenceEngineConfig(max_pages=max(1, max_tokens // ps), max_seqs=max_seqs, page_size=ps, max_pages_per_seq=16, compute_dtype="float32")
    cache = make_cache(model, cfg)
    runner = ModelRunner(model, cache, env)
    live, out = {}, {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if e["id"] not in live:
                live[e["id"]] = cache.open(e["id"])
            entries.append(StepEntry(live[e["id"]], e["tokens"], e["want"]))
        logits = runner.step(entries)
        cache.check_invariants()
        if after_step is not None:
            after_step(cache, live)
        if logits.shape[0]:
            out[s["step"]] = logits
        for rid in s["end"]:
            cache.close(live.pop(rid))
    cache.check_invariants()
    assert all(g.pool.n_free == g.pool.n_pages for g in cache.groups)
    return out, cache


@pytest.mark.parametrize("mode", ["whole", "singles", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(setup, mode):
    raw, W, model, env, reqs, plain = setup
    steps = {"whole": TR.trace_whole, "singles": TR.trace_prefill_then_singles, "portions": TR.trace_portions,
             "mixed": lambda r: TR.trace_mixed(r, seed=4)}[mode](reqs)
    TR.number(steps)
    got, _ = replay(model, env, steps, TR.peak_tokens(steps))
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    assert set(got) == set(want)
    for k in want:
        torch.testing.assert_close(got[k].double(), want[k], rtol=2e-4, atol=2e-4)


def test_the_registry_finds_the_architecture_and_readers_share_their_owners_unit(tmp_path):
    raw, W, model, env, config = build("A", tmp_path)
    assert isinstance(config, TativikConfig) and config.model_type_name == "tativik"
    assert LmConfig.from_dict(config.to_hf_config()) == config
    assert [b.kind for b in model.blocks] == ["gated_sandwich"] * 5
    # layers 1 and 3 read the unit that layer 0 writes; every other layer has a unit of its own
    assert [(e.cache, e.writes_cache) for e in model.plan] == [(0, True), (0, False), (1, True), (0, False), (2, True)]
    reqs = dict(model.cache_requirements())
    # the unit keeps what its widest reader sees (37 positions), the latent and the rotated key part as the key, the latent as the value
    assert reqs[0] == PagedKv(1, 32, 37, value_dim=24)
    assert reqs[1] == SlotState((2, 16, 16), "float32") and reqs[2] == SlotState((4, 8, 8), "float32")
    assert [b.mixer.window for b in model.blocks if hasattr(b.mixer, "window")] == [24, 37, 9]
    # the inner size of the decay's map is what the tensors say: the written configuration does not name it
    assert "decay_rank" not in config.layers[2]["mixer"] and model.blocks[2].mixer.rank == 8 and model.blocks[4].mixer.rank == 5
    raw_b, _, model_b, _, _ = build("B", tmp_path)
    assert dict(model_b.cache_requirements())[2] == PagedKv(1, 64, None, value_dim=32)  # a reader without a window: everything is kept


def test_the_residual_stream_after_every_layer(tmp_path):
    import levanter_amd.parts.gated_block as GB

    raw, W, model, env, _ = build("A", tmp_path)
    toks = TR.random_requests(raw["vocab"], [29], 3)["r0"]
    _, want = P.forward(raw, W, toks, True)
    got = []
    orig = GB.GatedSandwichBlock.forward

    def fwd(self, x, ctx, unit, wc):
        orig(self, x, ctx, unit, wc)
        assert ctx.pending is not None  # the last sublayer's write waits for the next norm
        ctx.settle()
        got.append(x.clone())

    GB.GatedSandwichBlock.forward = fwd
    try:
        cache = make_cache(model, InferenceEngineConfig(max_pages=8, max_seqs=2, page_size=16, max_pages_per_seq=8, compute_dtype="float32"))
        ModelRunner(model, cache, env).step([StepEntry(cache.open("a"), toks, [])])
    finally:
        GB.GatedSandwichBlock.forward = orig
    assert len(got) == len(want) == 5
    for g, w in zip(got, want):
        torch.testing.assert_close(g.double(), w, rtol=1e-4, atol=1e-4)


def test_windowed_groups_give_pages_back_and_take_used_ones(tmp_path):
    """A request of 100 tokens in portions: the group whose widest reader sees 37 positions never holds more than that window and
    a portion need, and pages freed behind the window are handed out again."""
    raw, W, model, env, _ = build("A", tmp_path)
    reqs = TR.random_requests(raw["vocab"], [100, 60], 9)
    steps = TR.number(TR.trace_portions(reqs, sizes=[7, 2, 13, 3, 5]))
    seen = {}

    def after(cache, live):
        for g in cache.groups:
            w = g.requirement.window
            for rid, h in live.items():
                held = len(g.pages_held(h.slot))
                first = max(0, h.length - w + 1) // 16
                assert held == -(-h.length // 16) - first
                seen[w] = max(seen.get(w, 0), held)

    got, cache = replay(model, env, steps, 128, after_step=after)
    assert seen[37] <= 4
    plain = {rid: P.plain_logits(W, raw, t) for rid, t in reqs.items()}
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    for k in want:
        torch.testing.assert_close(got[k].double(), want[k], rtol=2e-4, atol=2e-4)


def test_a_slot_that_is_used_again_starts_from_zero_state(tmp_path):
    """Two requests one after the other in an engine of one slot: the second finds the first one's state in its slot and pages."""
    raw, W, model, env, _ = build("B", tmp_path)
    reqs = TR.random_requests(raw["vocab"], [40, 23], 2)
    steps = TR.number(TR.trace_prefill_then_singles(reqs, n_single=5))
    got, _ = replay(model, env, steps, 64, max_seqs=1)
    plain = {rid: P.plain_logits(W, raw, t) for rid, t in reqs.items()}
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    for k in want:
        torch.testing.assert_close(got[k].double(), want[k], rtol=2e-4, atol=2e-4)


def test_bad_configurations_and_checkpoints_are_refused(tmp_path):
    raw, _ = TAT["A"]

    def broken(change):
        c = copy.deepcopy(raw)
        change(c)
        return c

    cases = [
        lambda c: c["layers"][0].update(type="attention"),
        lambda c: c["layers"][0]["mixer"].pop("kv_rank"),
        lambda c: c["layers"][0]["mixer"].pop("q_rank"),
        lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7),
        lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10),
        lambda c: c["layers"][0]["mixer"]["mask"].update(size=0),
        lambda c: c["layers"][1]["mixer"].update(kv_from=1),  # itself
        lambda c: c["layers"][1]["mixer"].update(kv_from=2),  # a later layer
        lambda c: c["layers"][3]["mixer"].update(kv_from=1),  # a layer that has no latent of its own
        lambda c: c["layers"][3]["mixer"].update(kv_from=2),  # a recurrent layer
        lambda c: c["layers"][1]["mixer"].update(kv_rank=16),  # not the owner's
        lambda c: c["layers"][1]["mixer"]["rot"].update(base=7.0),
        lambda c: c["layers"][0]["mlp"].update(kind="dense"),
        lambda c: c["layers"][0]["mlp"]["router"].update(top=5),  # more than the kept groups hold
        lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3),
        lambda c: c["layers"][2]["mixer"].pop("heads"),
        lambda c: c["norm"].update(groups=3),
        lambda c: c.pop("norm"),
        lambda c: c.pop("width"),
    ]
    for i, change in enumerate(cases):
        with pytest.raises(ConfigError):
            LmConfig.from_dict(broken(change))
            pytest.fail(f"case {i} was accepted")
    # a checkpoint that lacks a tensor, has one too many (a latent of its own in a layer that reads another's) and one of the wrong shape
    W = P.random_weights(raw, 1)
    W2 = dict(W)
    del W2["l2.mix.w0"]
    W2["l1.mix.dkv"] = torch.zeros(32, 64, dtype=torch.float64)
    W2["l0.mix.sink"] = torch.zeros(3, dtype=torch.float64)
    d = P.write_folder(raw, W2, str(tmp_path / "bad"), torch.float32)
    env = BuildEnv(torch.float32, torch.device("cpu"), EmulatedKernels())
    with pytest.raises(WeightsError) as e:
        load_model(d, env)
    assert e.value.missing == ["l2.mix.w0"] and e.value.unexpected == ["l1.mix.dkv"] and len(e.value.wrong_shape) == 1
    # the two matrices of the decay's map must agree on their inner size
    W3 = dict(W)
    W3["l2.mix.w1"] = torch.zeros(7, 64, dtype=torch.float64)
    d = P.write_folder(raw, W3, str(tmp_path / "bad2"), torch.float32)
    with pytest.raises(ValueError):
        load_model(d, env)


# ---- the plain implementation's mechanisms against direct statements ------------------------------------------------------
def test_group_norm_is_the_rms_norm_of_each_part():
    x = torch.randn(5, 12, dtype=torch.float64)
    w = torch.randn(12, dtype=torch.float64)
    got = P.group_rms_norm(x, w, 3, 1e-5)
    for g in range(3):
        part = x[:, 4 * g:4 * g + 4]
        torch.testing.assert_close(got[:, 4 * g:4 * g + 4], part / torch.sqrt((part ** 2).mean(-1, keepdim=True) + 1e-5) * w[4 * g:4 * g + 4])
    torch.testing.assert_close(P.group_rms_norm(x, w, 1, 1e-5), P.rms_norm(x, w, 1e-5))


def test_rotation_pairs_a_dimension_with_the_one_half_the_rotated_size_ahead():
    v = torch.zeros(1, 10, dtype=torch.float64)
    v[0, 1] = 1.0  # dimension 1 of a rotated size of 6 is paired with dimension 4; dimensions 6 .. 9 never turn
    v[0, 7] = 2.0
    out = P.rotate_half(v, torch.tensor([3]), 6, 100.0)
    a = 3 * 100.0 ** (-2.0 / 6)
    want = torch.zeros(10, dtype=torch.float64)
    want[1], want[4], want[7] = math.cos(a), math.sin(a), 2.0
    torch.testing.assert_close(out[0], want)
    q, k = torch.randn(2, 1, 8, dtype=torch.float64)  # scores depend on the distance alone
    s = [float((P.rotate_half(q, torch.tensor([p + 5]), 8, 50.0) * P.rotate_half(k, torch.tensor([p]), 8, 50.0)).sum()) for p in (0, 7, 300)]
    assert abs(s[0] - s[1]) < 1e-9 and abs(s[0] - s[2]) < 1e-9


def test_window_and_sink():
    ok = P.window_visible(6, 3)
    assert ok.tolist() == [[j <= i and i - j < 3 for j in range(6)] for i in range(6)]
    s = torch.tensor([[[0.0, 0.0], [1.0, 2.0]]], dtype=torch.float64)
    w = P.softmax_with_sink(s, P.window_visible(2, None), torch.tensor([0.5], dtype=torch.float64))
    assert abs(float(w[0, 0, 0]) - 1 / (1 + math.exp(0.5))) < 1e-12 and float(w[0, 0, 1]) == 0.0
    den = math.exp(1) + math.exp(2) + math.exp(0.5)
    torch.testing.assert_close(w[0, 1], torch.tensor([math.exp(1) / den, math.exp(2) / den], dtype=torch.float64))


def test_the_delta_rule_by_hand():
    """One head of two channels, two tokens: the second token's state from the first one's by the rule, written out."""
    r = torch.tensor([[[1.0, 0.0]], [[0.5, 2.0]]], dtype=torch.float64)
    k = torch.tensor([[[3.0, 4.0]], [[0.0, 2.0]]], dtype=torch.float64)
    v = torch.tensor([[[1.0, -1.0]], [[2.0, 0.5]]], dtype=torch.float64)
    w = torch.tensor([[[0.9, 0.8]], [[0.5, 0.7]]], dtype=torch.float64)
    a = torch.tensor([[[0.2, 0.3]], [[1.0, 0.4]]], dtype=torch.float64)
    o, S = P.delta_rule_scan(r, k, v, w, a)
    S1 = torch.outer(k[0, 0], v[0, 0])  # from zero: only the write
    torch.testing.assert_close(o[0, 0], S1.T @ r[0, 0])
    u = k[1, 0] / math.sqrt(4.0 + 1e-6)
    S2 = torch.diag(w[1, 0]) @ S1 - torch.outer(a[1, 0] * u, u @ S1) + torch.outer(k[1, 0], v[1, 0])
    torch.testing.assert_close(S[0], S2)
    torch.testing.assert_close(o[1, 0], S2.T @ r[1, 0])
    # carried state: two tokens at once equal one after the other
    o1, Sa = P.delta_rule_scan(r[:1], k[:1], v[:1], w[:1], a[:1])
    o2, Sb = P.delta_rule_scan(r[1:], k[1:], v[1:], w[1:], a[1:], Sa)
    torch.testing.assert_close(torch.cat([o1, o2]), o)
    torch.testing.assert_close(Sb, S)


def test_the_router_by_hand():
    """Eight experts in four groups of two, two groups kept, two experts used; the correction changes the choice, not the weights;
    a group with one very good expert loses to one with two good ones; choice scores below zero still beat an excluded expert."""
    inv = lambda s: math.log(s / (1 - s))
    s = [0.9, 0.1, 0.6, 0.55, 0.5, 0.45, 0.2, 0.3]
    z = torch.tensor([[inv(x) for x in s]], dtype=torch.float64)
    none = torch.zeros(8, dtype=torch.float64)
    chosen, weights = P.route(z, none, 2, 4, 2)
    # group scores 1.0, 1.15, 0.95, 0.5: groups 1 and 0 are kept; the winners are experts 0 and 2
    assert chosen.tolist() == [[0, 2]]
    torch.testing.assert_close(weights, torch.tensor([[0.9, 0.6]], dtype=torch.float64))
    corr = torch.tensor([-0.5, 0.0, 0.0, 0.0, 0.3, 0.3, 0.0, 0.0], dtype=torch.float64)
    chosen, weights = P.route(z, corr, 2, 4, 2)
    # choice scores 0.4, 0.1, 0.6, 0.55, 0.8, 0.75, 0.2, 0.3: groups 2 (1.55) and 1 (1.15) are kept; winners 4 and 5, weights without the correction
    assert chosen.tolist() == [[4, 5]]
    torch.testing.assert_close(weights, torch.tensor([[0.5, 0.45]], dtype=torch.float64))
    corr = torch.tensor([-2.0, -2.0, -2.0, -2.0, -2.0, -2.0, -1.5, -1.9], dtype=torch.float64)
    # all choice scores negative (-1.1 -1.9 | -1.4 -1.45 | -1.5 -1.55 | -1.3 -1.6): groups 1 (-2.85) and 3 (-2.9) are kept, and their three
    # best experts win although expert 0 of an excluded group has the best score of all (excluded means minus infinity, not zero)
    chosen, _ = P.route(z, corr, 3, 4, 2)
    assert chosen.tolist() == [[6, 2, 3]]
    chosen, _ = P.route(z, none, 3, 1, 1)  # one group: the plain top three
    assert chosen.tolist() == [[0, 2, 3]]
