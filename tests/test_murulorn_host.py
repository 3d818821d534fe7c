"""Murulorn through the engine's host side (configuration, weights by name, pages with windows, state slots, batching,
scheduler, sampling) on the CPU, with torch stand-ins for the kernels, against the plain implementation. The kernels
themselves are tested on the GPU (test_murulorn_gpu.py)."""
import copy
import math
import random

import pytest
import torch

import plain_murulorn as P
from murulorn_helpers import (CONFIGS, greedy, make_model, make_weights, plain_logits, public, rel_err, replay,
                              single_layer, write_model)
from torch_ops import TorchOps

from lmsf_amd.config import ConfigError, load_model_config, resolve_architecture
from lmsf_amd.engine import EngineArgs, LLMEngine, StepEntry, load_engine_core
from lmsf_amd.sampling import SamplingParams
from lmsf_amd.weights.loader import WeightsError

TOL = 3e-5
SMALL = ("A", "B", "C", "D")


def build(tmp_path, which, pages=24, block=8, seed=0, **kw):
    folder, cfg, w = make_model(tmp_path, which, seed, spread=kw.pop("spread", 1.0), weights=kw.pop("weights", None))
    core = load_engine_core(folder, dtype="float32", block_size=block, num_pages=pages, max_model_len=pages * block,
                            device="cpu", ops=TorchOps(), max_num_seqs=kw.pop("slots", 4), **kw)
    return core, cfg, w


def agrees(got, cfg, w, toks, ref=None):
    """float32: within TOL of the plain implementation in float64, or within three times what float32 rounding costs
    the plain implementation itself where that is more (several passes through a loop add up)."""
    ref = plain_logits(cfg, w, toks) if ref is None else ref
    tol = max(TOL, 3 * rel_err(plain_logits(cfg, w, toks, dtype=torch.float32), ref))
    return rel_err(got, ref) < tol


def tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def test_the_architecture_is_found_by_its_name():
    assert resolve_architecture({"architecture": "Murulorn"}).name == "Murulorn"


# ---------------------------------------------------------------- the plain implementation's own mechanisms


def test_plain_pair_rows_hash_the_token_before_and_the_token():
    assert P.bigram_rows([3, 5, 5, 0], 7, 4, 3) == [7, (3 * 4 + 5 * 3) % 7, (5 * 4 + 5 * 3) % 7, (5 * 4) % 7]
    assert P.bigram_rows([9], 1, 2, 3) == [1]


def test_plain_rotations_pair_as_they_say_and_turn_back():
    x = torch.arange(1.0, 9.0, dtype=torch.float64).reshape(1, 1, 8)
    pos = torch.tensor([3])
    a = P.turn_pairs(x, pos, 4, 10.0, True)[0, 0]
    b = P.turn_pairs(x, pos, 4, 10.0, False)[0, 0]
    f = [1.0, 10.0 ** -0.5]
    for i in range(2):
        c, s = math.cos(3 * f[i]), math.sin(3 * f[i])
        assert abs(a[2 * i] - (x[0, 0, 2 * i] * c - x[0, 0, 2 * i + 1] * s)) < 1e-12
        assert abs(a[2 * i + 1] - (x[0, 0, 2 * i + 1] * c + x[0, 0, 2 * i] * s)) < 1e-12
        assert abs(b[i] - (x[0, 0, i] * c - x[0, 0, i + 2] * s)) < 1e-12
        assert abs(b[i + 2] - (x[0, 0, i + 2] * c + x[0, 0, i] * s)) < 1e-12
    assert torch.equal(a[4:], x[0, 0, 4:]) and torch.equal(b[4:], x[0, 0, 4:])
    back = P.turn_pairs(P.turn_pairs(x, pos, 8, 50.0, True), pos, 8, 50.0, True, sign=-1.0)
    assert (back - x).abs().max() < 1e-12


def test_plain_delta_rule_writes_what_it_reads_back():
    """With no decay and beta 1 a unit key's value is replaced outright: reading with the same key gives the value
    just written, whatever was there; with a decay g the old memory enters the difference times g."""
    g0 = torch.Generator().manual_seed(3)
    k = torch.nn.functional.normalize(torch.randn((2, 1, 5), generator=g0, dtype=torch.float64), dim=-1)
    v = torch.randn((2, 1, 3), generator=g0, dtype=torch.float64)
    ones = torch.ones((2, 1, 5), dtype=torch.float64)
    o = P.delta_rule(k, k, v, torch.ones((2, 1), dtype=torch.float64), ones)
    assert (o - v).abs().max() < 1e-12
    g = torch.rand((2, 1, 5), generator=g0, dtype=torch.float64)
    beta = torch.rand((2, 1), generator=g0, dtype=torch.float64)
    q = torch.randn((2, 1, 5), generator=g0, dtype=torch.float64)
    o = P.delta_rule(q, k, v, beta, g)
    S1 = beta[0, 0] * torch.outer(k[0, 0], v[0, 0])
    Sd = g[1, 0][:, None] * S1
    S2 = Sd + torch.outer(k[1, 0], beta[1, 0] * (v[1, 0] - Sd.T @ k[1, 0]))
    assert (o[0, 0] - S1.T @ q[0, 0]).abs().max() < 1e-12 and (o[1, 0] - S2.T @ q[1, 0]).abs().max() < 1e-12


def test_plain_choice_stays_within_the_best_groups():
    s = torch.tensor([[0.05, 0.30, 0.10, 0.02, 0.25, 0.28]])       # groups of two: bests 0.30, 0.10, 0.28
    assert sorted(P.choose_experts(s, 2, 3, 2)[0].tolist()) == [1, 5]
    assert sorted(P.choose_experts(s, 3, 3, 2)[0].tolist()) == [1, 4, 5]      # 2 (0.10) lies in a group that is dropped
    assert sorted(P.choose_experts(s, 3, 1, 1)[0].tolist()) == [1, 4, 5]
    assert sorted(P.choose_experts(s, 2, 3, 1)[0].tolist()) == [0, 1]


def test_plain_attention_sees_values_turned_by_the_distance(tmp_path):
    """Turning a value by its own position and the sum back by the query's equals turning every value by j - i."""
    cfg = single_layer("B", 1)
    w = make_weights(cfg, 4)
    m = cfg["layers"][0]["mixer"]
    T, W = 9, cfg["width"]
    h = torch.randn((T, W), generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    tw = {k: v.double() for k, v in w.items()}
    got = P.attention(m, tw, "l0.mix", h, 1e-6, None)
    # by hand, for the last position
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (P.rms(h @ tw["l0.mix.q"].T, 1e-6) * tw["l0.mix.q.norm"]).view(T, H, d)
    k = (P.rms(h @ tw["l0.mix.k"].T, 1e-6) * tw["l0.mix.k.norm"]).view(T, G, d)
    q, k = P.turn_pairs(q, pos, m["rot"]["dims"], m["rot"]["base"], True), P.turn_pairs(k, pos, m["rot"]["dims"], m["rot"]["base"], True)
    v = P.rms((h @ tw["l0.mix.v"].T).view(T, G, dv), 1e-6)
    i = T - 1
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        s = (k[:, g] @ q[i, hd]) * m["scale"]
        s = m["softcap"] * torch.tanh(s / m["softcap"])
        p = torch.softmax(s, 0)
        turned = P.turn_pairs(v[:, g:g + 1], pos - i, dv, m["rot"]["base"], True)[:, 0]
        heads.append((p[:, None] * turned).sum(0) * torch.sigmoid(h[i] @ tw["l0.mix.g"][hd]))
    want = torch.cat(heads) @ tw["l0.mix.o"].T
    assert (got[i] - want).abs().max() < 1e-10


# ---------------------------------------------------------------- the engine against the plain implementation


@pytest.mark.parametrize("which", SMALL)
def test_whole_prompt(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(45, cfg["vocab"], 1)
    out = core.executor.step([StepEntry("a", toks, list(range(len(toks))))])
    assert agrees(out, cfg, w, toks)


@pytest.mark.parametrize("index", range(4))
def test_every_kind_of_layer_alone(tmp_path, index):
    cfg = single_layer("A", index, keep_loop=index % 2 == 0)
    core, cfg, w = build(tmp_path, cfg)
    toks = tokens(30, cfg["vocab"], 11)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in (7, 2, 12, 1, 1, 1, 6)])["a"]
    assert agrees(got, cfg, w, toks)


@pytest.mark.parametrize("which", SMALL)
def test_portions_down_to_two_tokens_then_one_by_one(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(61, cfg["vocab"], 2)
    cuts = [3, 2, 8, 7, 2, 16, 9] + [1] * 14          # portions that end inside and on the edges of pages and windows
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    assert agrees(got, cfg, w, toks)
    core.storage.manager.check_invariants()


@pytest.mark.parametrize("which", SMALL)
def test_token_by_token_from_the_first(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(24, cfg["vocab"], 3)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    assert agrees(got, cfg, w, toks)


@pytest.mark.parametrize("which", SMALL)
def test_unequal_requests_together_with_pages_and_slots_used_again(tmp_path, which):
    core, cfg, w = build(tmp_path, which, pages=20, slots=3)     # 160 tokens of room, three state slots
    V = cfg["vocab"]
    reqs = {"a": tokens(70, V, 4), "b": tokens(1, V, 5), "c": tokens(33, V, 6), "d": tokens(90, V, 7),
            "e": tokens(5, V, 8)}
    steps = [[("a", 30), ("b", 1), ("c", 2)], [("a", 1), ("c", 17), ("e", 2)], [("c", 14), ("a", 38)], [("a", 1), ("e", 3)],
             [("d", 50)], [("d", 39)], [("d", 1)]]
    got = replay(core.executor, StepEntry, reqs, steps)
    for k, t in reqs.items():
        assert agrees(got[k], cfg, w, t), k
    mgr = core.storage.manager
    mgr.check_invariants()
    assert all(mgr.num_free_pages(g) == 20 for g in range(len(mgr.groups))) and mgr.num_free_state_slots() == 3


def test_a_request_that_sits_a_step_out_keeps_its_token_before(tmp_path):
    """The token before a step's first is state: a request that is left out of steps while others run, and another
    that takes the slot a finished one held, still hash the right pair."""
    core, cfg, w = build(tmp_path, "D", slots=2)
    V = cfg["vocab"]
    reqs = {"a": tokens(12, V, 31), "b": tokens(9, V, 32), "c": tokens(7, V, 33)}
    steps = [[("a", 5)], [("b", 9)], [("c", 3)], [("a", 1)], [("c", 4)], [("a", 6)]]
    got = replay(core.executor, StepEntry, reqs, steps)
    for k, t in reqs.items():
        assert agrees(got[k], cfg, w, t), k


def test_every_pass_of_a_loop_has_pages_and_state_of_its_own(tmp_path):
    core, cfg, w = build(tmp_path, "A")
    runs = [e.layer for e in core.model.schedule]
    assert runs == [0, 1, 2, 1, 2, 3]
    pages = [b.k_pages.data_ptr() for b in core.model.bindings if b.k_pages is not None]
    states = [b.state.data_ptr() for b in core.model.bindings if b.state is not None]
    assert len(set(pages)) == 3 and len(set(states)) == 3


def test_a_window_gives_its_pages_back(tmp_path):
    core, cfg, w = build(tmp_path, "B", pages=30, block=4)
    assert sorted(g.spec.window for g in core.storage.groups) == [1, 7, 19]
    toks = tokens(100, cfg["vocab"], 9)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", 50)]] + [[("a", 1)]] * 50)
    assert agrees(got["a"], cfg, w, toks)
    assert all(core.storage.manager.num_free_pages(g) == 30 for g in range(3))


def test_keys_just_inside_and_just_outside_a_window_decide_or_do_not(tmp_path):
    """One layer of attention with a window of 11 and peaked scores: the plain implementation says that changing the
    token 10 back moves the last position's logits and that changing the token 11 back moves nothing (the pair row of
    the token behind it aside, which is why the token behind keeps its pair's row: multipliers of zero); the engine
    agrees with it on all three sequences, in a prompt and decoding."""
    cfg = single_layer("A", 1)
    cfg["embedding"] = {"bigram": {"buckets": 5, "mul_prev": 0, "mul_cur": 3}}
    folder, cfg, w = make_model(tmp_path, cfg, 5, spread=4.0)
    size = cfg["layers"][0]["mixer"]["mask"]["size"]
    base = tokens(40, cfg["vocab"], 12)
    inside, outside = list(base), list(base)
    inside[39 - (size - 1)] = (base[39 - (size - 1)] + 1) % cfg["vocab"]
    outside[39 - size] = (base[39 - size] + 1) % cfg["vocab"]
    ref = {k: plain_logits(cfg, w, t) for k, t in (("base", base), ("inside", inside), ("outside", outside))}
    spread = float(ref["base"].double().std())
    assert float((ref["inside"][-1] - ref["base"][-1]).abs().max()) > 100 * TOL * spread
    assert float((ref["outside"][-1] - ref["base"][-1]).abs().max()) == 0.0
    for cuts in ([40], [30] + [1] * 10, [27, 2, 11]):
        core = load_engine_core(folder, dtype="float32", block_size=4, num_pages=12, max_model_len=48, device="cpu",
                                ops=TorchOps(), max_num_seqs=2)
        for k, t in (("base", base), ("inside", inside), ("outside", outside)):
            got = replay(core.executor, StepEntry, {k: t}, [[(k, c)] for c in cuts])[k]
            assert agrees(got, cfg, w, t, ref[k]), (k, cuts)


def test_a_far_token_reaches_the_last_through_the_memory(tmp_path):
    """The delta rule's memory with slow decays keeps the first token of 150: it moves the last logits, and the engine
    carries it through portions, single tokens and a slot that another request has used before."""
    cfg = single_layer("C", 1)
    w = make_weights(cfg, 6)
    w["l0.mix.A_log"][:] = -6.0                        # decays close to 1
    folder, cfg, w = make_model(tmp_path, cfg, 6, weights=w)
    a = tokens(150, cfg["vocab"], 13)
    b = [(a[0] + 1) % cfg["vocab"]] + a[1:]
    ra, rb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    assert float((ra[-1] - rb[-1]).abs().max()) > 100 * TOL * float(ra.double().std())
    core = load_engine_core(folder, dtype="float32", block_size=8, num_pages=4, max_model_len=160, device="cpu",
                            ops=TorchOps(), max_num_seqs=1)
    for k, t, ref in (("a", a, ra), ("b", b, rb)):
        got = replay(core.executor, StepEntry, {k: t}, [[(k, c)] for c in [64, 3, 70] + [1] * 13])[k]
        assert agrees(got, cfg, w, t, ref), k


def test_greedy_generation_through_the_engine_and_its_scheduler(tmp_path):
    folder, cfg, w = make_model(tmp_path, "A", 2)
    prompts = [tokens(9, cfg["vocab"], 20), tokens(23, cfg["vocab"], 21), tokens(2, cfg["vocab"], 22)]
    want = [greedy(cfg, w, p, 6) for p in prompts]
    engine = LLMEngine(EngineArgs(model=folder, dtype="float32", block_size=8, num_gpu_blocks_override=16, max_num_seqs=2,
                                  max_model_len=120, prefill_chunk_size=8, max_num_batched_tokens=12, device="cpu"),
                       ops=TorchOps())
    for i, p in enumerate(prompts):
        engine.add_request(i, p, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    done = {}
    while engine.has_unfinished_requests():
        for out in engine.step():
            if out.finished:
                done[int(out.request_id)] = list(out.outputs[0].token_ids)
    assert [done[i] for i in range(3)] == want


# ---------------------------------------------------------------- configuration and weights


def test_the_ranks_come_from_the_tensors_shapes(tmp_path):
    folder, cfg, w = make_model(tmp_path, "A", 0)
    arch, parsed = load_model_config(folder)
    assert arch.name == "Murulorn"
    got = [(lay["mixer"]["decay_rank"], lay["mixer"]["gate_rank"]) for lay in parsed.layers if lay["type"] == "channel_delta"]
    assert got == [(5, 7), (8, 3)]
    assert "decay_rank" not in json_of(folder)["layers"][0]["mixer"]


def json_of(folder):
    import json
    import os
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def test_configuration_faults_name_their_key():
    def parse(cfg):
        return resolve_architecture(cfg).config_class.from_dict(public(cfg))

    for path, value, word in ((("layers", 1, "mixer", "rot", "dims"), 7, "dims"),
                              (("layers", 1, "mlp", "router", "top"), 9, "router"),
                              (("layers", 1, "mlp", "router", "groups", "keep"), 4, "groups"),
                              (("layers", 0, "type"), "retention", "type"),
                              (("layers", 1, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("loop", "stop"), 9, "loop"),
                              (("embedding", "bigram", "buckets"), 0, "buckets")):
        cfg = copy.deepcopy(CONFIGS["A"])
        at = cfg
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            parse(cfg)
    cfg = copy.deepcopy(CONFIGS["A"])
    del cfg["layers"][3]["mixer"]["mask"]
    with pytest.raises(ConfigError, match="mask"):
        parse(cfg)


def test_weight_faults_are_listed_by_name(tmp_path):
    cfg = CONFIGS["A"]
    w = make_weights(cfg, 0)
    del w["l1.mix.q.norm"], w["loop.in"]
    w["l2.mix.v.conv"] = w["l2.mix.v.conv"][:, :1]
    folder = write_model(str(tmp_path / "broken"), cfg, w)
    with pytest.raises(WeightsError) as e:
        load_engine_core(folder, dtype="float32", block_size=8, num_pages=4, device="cpu", ops=TorchOps())
    assert "l1.mix.q.norm" in e.value.missing and "loop.in" in e.value.missing
    assert any(n == "l2.mix.v.conv" for n, _, _ in e.value.wrong_shape)
