"""Zevetar through the engine's host side (configuration, weights by name, pages with windows, state slots, batching,
scheduler, sampling) on the CPU, with torch stand-ins for the kernels, against the plain implementation. The kernels
themselves are tested on the GPU (test_zevetar_gpu.py)."""
import copy
import math
import random

import pytest
import torch

import plain_zevetar as P
from torch_ops import TorchOps
from zevetar_helpers import CONFIGS, make_model, make_weights, plain_logits, rel_err, replay, single_layer, write_model

from lmsf_amd.config import ConfigError, resolve_architecture
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


def tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def test_the_architecture_is_found_by_its_name():
    assert resolve_architecture({"architecture": "Zevetar"}).name == "Zevetar"


# ---------------------------------------------------------------- the plain implementation's own mechanisms


def test_plain_yarn_frequencies_meet_both_ends_and_the_gain():
    f, gain = P.rotary_frequencies(16, 100.0, None, torch.float64)
    assert gain == 1.0 and torch.allclose(f, 100.0 ** (-torch.arange(8, dtype=torch.float64) / 8))
    sc = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 0.25}
    g, gain = P.rotary_frequencies(16, 100.0, sc, torch.float64)
    assert abs(gain - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    # fast pairs keep their frequency, slow ones are divided by the factor, those between lie between
    assert g[0] == f[0] and abs(g[-1] - f[-1] / 4.0) < 1e-15
    assert ((g <= f + 1e-15) & (g >= f / 4.0 - 1e-15)).all()


def test_plain_rotations_pair_as_they_say():
    x = torch.arange(1.0, 9.0, dtype=torch.float64).reshape(1, 1, 8)
    pos = torch.tensor([3])
    a = P.rotate(x, pos, 4, 10.0, None, True)[0, 0]
    b = P.rotate(x, pos, 4, 10.0, None, False)[0, 0]
    f = [1.0, 10.0 ** -0.5]
    for i in range(2):
        c, s = math.cos(3 * f[i]), math.sin(3 * f[i])
        u, v = x[0, 0, 2 * i], x[0, 0, 2 * i + 1]
        assert abs(a[2 * i] - (u * c - v * s)) < 1e-12 and abs(a[2 * i + 1] - (v * c + u * s)) < 1e-12
        u, v = x[0, 0, i], x[0, 0, i + 2]
        assert abs(b[i] - (u * c - v * s)) < 1e-12 and abs(b[i + 2] - (v * c + u * s)) < 1e-12
    assert torch.equal(a[4:], x[0, 0, 4:]) and torch.equal(b[4:], x[0, 0, 4:])


def test_plain_retention_is_the_sum_over_earlier_tokens():
    cfg = single_layer("A", 2)
    m = cfg["layers"][0]["mixer"]
    m.pop("rot")
    w = {k: v.double() for k, v in make_weights(cfg, 3).items()}
    T, W = 9, cfg["width"]
    h = torch.randn(T, W, dtype=torch.float64)
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["l0.mix.q"].T).reshape(T, H, d)
    k = (h @ w["l0.mix.k"].T).reshape(T, H, d) * d ** -0.5
    v = (h @ w["l0.mix.v"].T).reshape(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        for u in range(t + 1):
            for hh in range(H):
                o[t, hh] += m["decay"][hh] ** (t - u) * (q[t, hh] @ k[u, hh]) * v[u, hh]
    o = P.rms_norm(o, None, 1e-5).reshape(T, -1) * P.silu(h @ w["l0.mix.g"].T)
    want = o @ w["l0.mix.o"].T
    got = P.retention(h, m, w, "l0.mix.", 1e-5, torch.arange(T), None)
    assert (got - want).abs().max() < 1e-10


def test_plain_experts_weigh_the_input_not_the_output():
    cfg = single_layer("A", 1)
    mlp = cfg["layers"][0]["mlp"]
    w = {k: v.double() for k, v in make_weights(cfg, 4).items()}
    h = torch.randn(5, cfg["width"], dtype=torch.float64)
    got = P.routed_experts(h, mlp, w, "l0.mlp.", None)
    s = torch.sigmoid(h @ w["l0.mlp.router"].T)
    for n in range(5):
        want = torch.sigmoid(h[n] @ w["l0.mlp.shared.sg"][0]) * P.gated_ffn(h[n:n + 1], w, "l0.mlp.shared.", None)[0]
        for e in torch.argsort(-s[n])[:mlp["router"]["top"]].tolist():
            want = want + P.gated_ffn(s[n, e] * h[n:n + 1], w, "l0.mlp.e%d." % e, None)[0]
        assert (got[n] - want).abs().max() < 1e-10


# ---------------------------------------------------------------- the engine against the plain implementation


@pytest.mark.parametrize("which", SMALL)
def test_whole_prompt(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(45, cfg["vocab"], 1)
    out = core.executor.step([StepEntry("a", toks, list(range(len(toks))))])
    assert rel_err(out, plain_logits(cfg, w, toks)) < TOL


@pytest.mark.parametrize("index", range(4))
def test_every_kind_of_layer_alone(tmp_path, index):
    cfg = single_layer("A", index)
    core, cfg, w = build(tmp_path, cfg)
    toks = tokens(30, cfg["vocab"], 11)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in (7, 2, 12, 1, 1, 1, 6)])["a"]
    assert rel_err(got, plain_logits(cfg, w, toks)) < TOL


@pytest.mark.parametrize("which", SMALL)
def test_portions_down_to_two_tokens_then_one_by_one(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(61, cfg["vocab"], 2)
    cuts = [3, 2, 8, 7, 2, 16, 9] + [1] * 14          # portions that end inside and on the edges of pages and windows
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    assert rel_err(got, plain_logits(cfg, w, toks)) < TOL
    core.storage.manager.check_invariants()


@pytest.mark.parametrize("which", SMALL)
def test_token_by_token_from_the_first(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(24, cfg["vocab"], 3)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    assert rel_err(got, plain_logits(cfg, w, toks)) < TOL


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
        assert rel_err(got[k], plain_logits(cfg, w, t)) < TOL, k
    mgr = core.storage.manager
    mgr.check_invariants()
    assert all(mgr.num_free_pages(g) == 20 for g in range(len(mgr.groups))) and mgr.num_free_state_slots() == 3


def test_a_window_gives_its_pages_back_and_the_widest_reader_decides(tmp_path):
    """Layer 1 of "A" reads layer 0's latent with a window of 19, layer 0 itself sees 11: the pages stay for 19."""
    core, cfg, w = build(tmp_path, "A", pages=30, block=4)
    specs = [g.spec.window for g in core.storage.groups]
    assert sorted(s or 0 for s in specs) == [0, 19]
    toks = tokens(100, cfg["vocab"], 9)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", 50)]] + [[("a", 1)]] * 49 + [[("a", 1)]])
    assert rel_err(got["a"], plain_logits(cfg, w, toks)) < TOL
    windowed = [i for i, g in enumerate(core.storage.groups) if g.spec.window][0]
    # (released above: all free again; while it ran, at most the window's pages and one were held)
    assert core.storage.manager.num_free_pages(windowed) == 30


def test_keys_just_inside_and_just_outside_a_window_decide_or_do_not(tmp_path):
    """One layer of attention with a window of 11 and peaked scores: the plain implementation says that changing the
    token 10 back moves the last position's logits and that changing the token 11 back moves nothing; the engine
    agrees with it on all three sequences, in a prompt and decoding."""
    cfg = single_layer("A", 0)
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
            assert rel_err(got, ref[k]) < TOL, (k, cuts)


def test_a_far_token_reaches_the_last_through_a_decay_of_one(tmp_path):
    """Retention with a decay of 1 forgets nothing: the first token of 150 moves the last logits, and the engine
    carries it through portions, single tokens and a slot that another request has used before."""
    cfg = single_layer("B", 0)
    folder, cfg, w = make_model(tmp_path, cfg, 6)
    a = tokens(150, cfg["vocab"], 13)
    b = [(a[0] + 1) % cfg["vocab"]] + a[1:]
    ra, rb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    assert float((ra[-1] - rb[-1]).abs().max()) > 100 * TOL * float(ra.double().std())
    core = load_engine_core(folder, dtype="float32", block_size=8, num_pages=4, max_model_len=160, device="cpu",
                            ops=TorchOps(), max_num_seqs=1)
    for k, t, ref in (("a", a, ra), ("b", b, rb)):
        got = replay(core.executor, StepEntry, {k: t}, [[(k, c)] for c in [64, 3, 70] + [1] * 13])[k]
        assert rel_err(got, ref) < TOL, k


def test_greedy_generation_through_the_engine_and_its_scheduler(tmp_path):
    folder, cfg, w = make_model(tmp_path, "A", 2)
    prompts = [tokens(9, cfg["vocab"], 20), tokens(23, cfg["vocab"], 21), tokens(2, cfg["vocab"], 22)]
    want = [P.greedy(cfg, w, p, 6) for p in prompts]
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


# ---------------------------------------------------------------- faults are named


def test_configuration_faults_name_their_key():
    cfg = copy.deepcopy(CONFIGS["A"])
    cfg["layers"][1]["mixer"]["kv_from"] = 2
    with pytest.raises(ConfigError, match="kv_from"):
        resolve_architecture(cfg).config_class.from_dict(cfg)
    cfg = copy.deepcopy(CONFIGS["A"])
    cfg["layers"][2]["mixer"]["decay"] = [0.5]
    with pytest.raises(ConfigError, match="decay"):
        resolve_architecture(cfg).config_class.from_dict(cfg)
    cfg = copy.deepcopy(CONFIGS["A"])
    cfg["layers"][1]["mlp"]["router"]["top"] = 9
    with pytest.raises(ConfigError, match="top"):
        resolve_architecture(cfg).config_class.from_dict(cfg)
    cfg = copy.deepcopy(CONFIGS["A"])
    cfg["layers"][0]["type"] = "attention"
    with pytest.raises(ConfigError, match="type"):
        resolve_architecture(cfg).config_class.from_dict(cfg)


def test_weight_faults_are_listed_by_name(tmp_path):
    cfg = CONFIGS["C"]
    w = make_weights(cfg, 0)
    del w["l0.mlp.shared.sg"]
    w["l1.mix.q"] = w["l1.mix.q"][:-1]
    folder = write_model(str(tmp_path / "broken"), cfg, w)
    with pytest.raises(WeightsError) as e:
        load_engine_core(folder, dtype="float32", block_size=8, num_pages=4, device="cpu", ops=TorchOps())
    assert "l0.mlp.shared.sg" in e.value.missing and any(n == "l1.mix.q" for n, _, _ in e.value.wrong_shape)
