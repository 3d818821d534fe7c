"""Murulorn on the GPU: the new kernels alone against the plain implementation's function of the same mechanism, every
kind of layer alone and the whole model through the engine's step function in float32 and bfloat16 under the ways of
cutting a request into steps, keys at a window's edges and far away made to decide the logits, pages and state slots
used again, long decoding from graphs, configurations drawn at random, and generation through the entry point."""
import os
import random
import subprocess
from types import SimpleNamespace

import pytest
import torch

import plain_murulorn as P
from helpers import (random_tokens, replay_in_process, replay_with_program, trace_bulk_then_single, trace_mixed,
                     trace_portions, trace_whole)
from murulorn_helpers import (attn, bfloat16_limits, delta, dense, greedy, make_model, make_weights, model, moe,
                              plain_logits, rel_err, replay, single_layer, within)

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

DTYPES = [torch.float32, torch.bfloat16]
TOL_F32 = 3e-5


def ops():
    from lmsf_amd.ops import get_ops
    return get_ops()


def close(got, ref, dtype, scale=1.0):
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    err = float((got.double().cpu() - ref.double().cpu()).abs().max())
    assert err <= tol * max(scale, float(ref.double().abs().max())), (err, float(ref.double().abs().max()))


def check(got, ref, dtype, what, model_, yardstick=0.0):
    """float32: three times what float32 rounding costs the plain implementation itself, where that is more than
    TOL_F32 (``yardstick``: that cost as the caller has measured it on other requests of the same model; one request
    is one draw of the rounding errors, and how much a model amplifies them is the model's property); bfloat16: per
    position three times what rounding costs the plain implementation when it rounds what an engine may keep in 16
    bits."""
    cfg, w, toks = model_
    if dtype == "float32":
        tol = max(TOL_F32, 3 * max(yardstick, rel_err(plain_logits(cfg, w, toks, dtype=torch.float32), ref)))
        assert rel_err(got, ref) < tol, (what, rel_err(got, ref), tol)
    else:
        ok, worst = within(got, ref, bfloat16_limits(cfg, w, toks, ref))
        assert ok, (what, worst)


def batch_of(lens, slots, first_pos=None, ids=None, dev="cuda"):
    """What the kernels read of a step: segments of ``lens`` tokens in state slots ``slots``."""
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    first_pos = first_pos or [0] * len(lens)
    pos = [p0 + i for p0, n in zip(first_pos, lens) for i in range(n)]
    seg = [s for s, n in enumerate(lens) for _ in range(n)]
    i32 = dict(dtype=torch.int32, device=dev)
    return SimpleNamespace(n_segments=len(lens), seg_starts=torch.tensor(starts, **i32), state_slots=torch.tensor(slots, **i32),
                           seg_of_token=torch.tensor(seg, **i32), positions=torch.tensor(pos, **i32),
                           token_ids=torch.tensor(ids, **i32) if ids is not None else None,
                           host_seg_lens=list(lens), all_single=all(n == 1 for n in lens), replayed=False, aux={})


def memory_as_the_kernel_keeps_it(S):
    """[H, d, dv] -> the kernel's [H, ceil(dv / 4), d, 4], flat."""
    H, d, dv = S.shape
    pad = -dv % 4
    S = torch.nn.functional.pad(S, (0, pad))
    return S.reshape(H, d, (dv + pad) // 4, 4).permute(0, 2, 1, 3).reshape(-1)


def table_of(dims, base, n=400):
    i = torch.arange(dims // 2, dtype=torch.float64)
    ang = torch.arange(n, dtype=torch.float64)[:, None] * (float(base) ** (-2.0 * i / dims))[None, :]
    return torch.cat([torch.cos(ang), torch.sin(ang)], 1).float().contiguous().cuda()


# ---------------------------------------------------------------- kernels alone


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,lens", [(3, 1, 8, 20, [5, 1, 17]), (2, 2, 64, 96, [70, 2, 9]), (1, 1, 24, 8, [1, 1, 1]),
                                            (4, 2, 128, 40, [33, 64]), (2, 1, 20, 133, [16, 47, 8]),
                                            (2, 2, 256, 16, [20, 2]), (6, 3, 33, 65, [9])])
def test_the_delta_rule_against_the_recurrence(dtype, H, G, d, dv, lens):
    """Segments continued from states that an earlier step left, in scattered slots, against the plain recurrence in
    float64: keys of 8 to 256 entries (every number of rows a lane holds), values that fill a block of columns, run
    over it and leave most of it empty."""
    o = ops()
    g = torch.Generator().manual_seed(H * 100 + d)
    slots = [2, 0, 3][:len(lens)]
    N = sum(lens)
    width = 2 * G * d + H * dv + 5
    p = (torch.randn((N, width), generator=g) * 0.7).to(dtype)
    a = torch.randn((N, H * d + 3), generator=g)
    b = torch.randn((N, H + 2), generator=g) * 2
    dt_bias, a_log = torch.randn((H * d,), generator=g), torch.rand((H,), generator=g) * 2 - 1.5
    mem = [torch.randn((H, d, dv), generator=g) * 0.3 for _ in range(5)]
    mem[0] = torch.zeros((H, d, dv))
    floats = o.gated_delta_state_floats(H, d, dv)
    assert floats == H * ((dv + 3) // 4) * d * 4
    state0 = torch.randn((5, floats + 3), generator=g)
    for i in range(5):
        state0[i, :floats] = memory_as_the_kernel_keeps_it(mem[i])
    pd = p.double()
    rep = H // G
    q = pd[:, 3:3 + G * d].reshape(N, G, d)
    k = pd[:, 3 + G * d:3 + 2 * G * d].reshape(N, G, d)
    v = pd[:, 3 + 2 * G * d:3 + 2 * G * d + H * dv].reshape(N, H, dv)
    q = (q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5).repeat_interleave(rep, 1)
    k = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(rep, 1)
    beta = torch.sigmoid(b[:, :H].double())
    decay = torch.exp(-torch.exp(a_log.double())[None, :, None] * torch.nn.functional.softplus(
        a[:, :H * d].double() + dt_bias.double()).reshape(N, H, d))
    want = torch.empty((N, H * dv), dtype=torch.float64)
    st = [m.double() for m in mem]
    at = 0
    for n, slot in zip(lens, slots):
        S = st[slot].clone()
        for t in range(at, at + n):
            S = S * decay[t][:, :, None]
            u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            want[t] = torch.einsum("hdv,hd->hv", S, q[t]).reshape(-1)
        st[slot] = S
        at += n
    # the recurrence itself, from one segment and a zero state, is the plain implementation's function
    one = P.delta_rule(q[:lens[0]], k[:lens[0]], v[:lens[0]], beta[:lens[0]], decay[:lens[0]])
    if slots[0] == 0:
        assert (one.reshape(lens[0], -1) - want[:lens[0]]).abs().max() < 1e-9
    state = state0.cuda()
    got = o.gated_delta(p.cuda(), 3, 3 + G * d, 3 + 2 * G * d, a.cuda(), dt_bias.cuda(), a_log.cuda(), b.cuda(), state,
                        batch_of(lens, slots), H, G, d, dv, d ** -0.5, 1e-6)
    assert got.dtype == torch.float32
    assert float((got.double().cpu() - want).abs().max()) <= 3e-5 * max(1.0, float(want.abs().max()))
    for i in range(5):
        want_i = memory_as_the_kernel_keeps_it(st[i])
        assert float((state.cpu()[i, :floats].double() - want_i).abs().max()) <= 3e-5 * max(1.0, float(want_i.abs().max()))
    assert torch.equal(state.cpu()[:, floats:], state0[:, floats:])        # what lies behind is not touched
    assert torch.equal(state.cpu()[1], state0[1]) and torch.equal(state.cpu()[4], state0[4])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dv,N,act", [(3, 20, 7, "sigmoid"), (1, 128, 300, "sigmoid"), (5, 66, 33, "silu")])
def test_heads_over_their_root_mean_square_with_weight_and_gate(dtype, H, dv, N, act):
    g = torch.Generator().manual_seed(dv)
    raw = torch.randn((N, H * dv), generator=g) * 3
    gate = torch.randn((N, H * dv + 4), generator=g).to(dtype)
    wt = 1 + 0.2 * torch.randn((dv,), generator=g)
    x = raw.double().reshape(N, H, dv)
    gd = gate[:, :H * dv].double().reshape(N, H, dv)
    want = P.rms(x, 1e-5) * wt.double() * (torch.sigmoid(gd) if act == "sigmoid" else gd * torch.sigmoid(gd))
    got = ops().head_rms_gate(raw.cuda(), H, dv, 1e-5, wt.cuda(), gate.cuda(), dtype, act)
    close(got, want.reshape(N, -1), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("H,G,d,dv,rot,ps", [(4, 2, 12, 8, 6, 4), (1, 1, 64, 64, 64, 16), (6, 3, 20, 36, 2, 8),
                                              (2, 1, 128, 96, 32, 16)])
def test_queries_keys_and_values_made_ready(dtype, interleaved, H, G, d, dv, rot, ps):
    """The norms over whole projections, both rotations and the pages against the plain functions, rows at page
    borders, a token that is not stored, and the turn back after attention."""
    o = ops()
    g = torch.Generator().manual_seed(d + dv)
    N, pages = 9, 5
    D = (max(d, dv) + 15) // 16 * 16
    p = torch.randn((N, (H + G) * d + G * dv + H + 3), generator=g).to(dtype)
    wq, wk = 1 + 0.2 * torch.randn((H * d,), generator=g), 1 + 0.2 * torch.randn((G * d,), generator=g)
    pos = torch.tensor([0, 1, 2, 3, 4, 17, 18, 399, 7])
    slots = torch.tensor([0, 1, ps - 1, ps, 2 * ps + 1, 3 * ps, 4 * ps + ps - 1, -1, 5], dtype=torch.int32)
    pd = p.double()
    q = (P.rms(pd[:, :H * d], 1e-5) * wq.double()).reshape(N, H, d)
    k = (P.rms(pd[:, H * d:(H + G) * d], 1e-5) * wk.double()).reshape(N, G, d)
    v = P.rms(pd[:, (H + G) * d:(H + G) * d + G * dv].reshape(N, G, dv), 1e-5)
    q, k = P.turn_pairs(q, pos, rot, 50.0, interleaved), P.turn_pairs(k, pos, rot, 50.0, interleaved)
    v = P.turn_pairs(v, pos, dv, 50.0, interleaved)
    kp = torch.full((pages, G, ps, D), 9.0, dtype=dtype, device="cuda")
    vp = torch.full((pages, G, D, ps), 9.0, dtype=dtype, device="cuda")
    pc = p.cuda()
    qa = o.attn_prepare_normed(pc[:, :H * d], pc[:, H * d:(H + G) * d], pc[:, (H + G) * d:], H, G, d, dv, D, pos.int().cuda(),
                               slots.cuda(), kp, vp, q_weight=wq.cuda(), k_weight=wk.cuda(), eps=1e-5,
                               table=table_of(rot, 50.0), table_v=table_of(dv, 50.0), interleaved=interleaved, v_norm=True)
    qa = qa.reshape(N, H, D)
    close(qa[..., :d], q, dtype)
    assert float(qa[..., d:].abs().max()) == 0.0 if D > d else True
    for t in range(N):
        s = int(slots[t])
        if s < 0:
            continue
        close(kp[s // ps, :, s % ps, :d], k[t], dtype)
        close(vp[s // ps, :, :dv, s % ps], v[t], dtype)
        assert float(kp[s // ps, :, s % ps, d:].abs().max() if D > d else 0.0) == 0.0
        assert float(vp[s // ps, :, dv:, s % ps].abs().max() if D > dv else 0.0) == 0.0
    used = {int(s) for s in slots if s >= 0}
    free = [s for s in range(pages * ps) if s not in used]
    assert all(float((kp[s // ps, :, s % ps] - 9.0).abs().max()) == 0.0 for s in free)    # nothing else is written
    # after attention: back by the position, times the head's gate
    a = torch.randn((N, H * D), generator=g).to(dtype)
    gate = pc[:, (H + G) * d + G * dv:]
    want = P.turn_pairs(a.double().reshape(N, H, D)[..., :dv], pos, dv, 50.0, interleaved, sign=-1.0) \
        * torch.sigmoid(gate[:, :H].double().cpu())[:, :, None]
    got = o.attn_finish(a.cuda(), D, H, dv, pos.int().cuda(), gate=gate, table_v=table_of(dv, 50.0), interleaved=interleaved)
    close(got, want.reshape(N, -1), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cap", [0.0, 3.0, 30.0])
def test_attention_bounds_its_scores(dtype, cap):
    """All three attention kernels (the general one in float32; the prefill and decode kernels of the matrix cores in
    bfloat16) with scores far above the cap, a window, and requests of one and of many tokens."""
    from torch_ops import TorchOps
    o = ops()
    g = torch.Generator().manual_seed(5)
    H, G, D, ps, window = 4, 2, 64, 16, 37
    lens = [70, 1, 1, 130]
    first = [0, 55, 3, 20]
    pages = 32
    kp = (torch.randn((pages, G, ps, D), generator=g) * 1.5).to(dtype)
    vp = torch.randn((pages, G, D, ps), generator=g).to(dtype)
    N = sum(lens)
    q = (torch.randn((N, H * D), generator=g) * 1.5).to(dtype)
    tables = torch.stack([torch.randperm(pages, generator=g)[:10] for _ in lens]).int()
    b = batch_of(lens, [0, 1, 2, 3], first, dev="cpu")
    want = TorchOps().paged_attention(q.float(), kp.float(), vp.float(), tables, b.seg_of_token, b.positions, H, G, D, 0.2,
                                      window, softcap=cap)
    bc = batch_of(lens, [0, 1, 2, 3], first)
    got = o.paged_attention(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), bc.seg_of_token, bc.positions, H, G, D, 0.2,
                            window, softcap=cap)
    close(got, want, dtype)
    if cap:
        plain = TorchOps().paged_attention(q.float(), kp.float(), vp.float(), tables, b.seg_of_token, b.positions, H, G, D,
                                           0.2, window)
        assert float((plain - want).abs().max()) > 0.05            # the cap matters at these scores


@pytest.mark.parametrize("E,top,groups,keep,N", [(6, 2, 3, 2, 7), (64, 6, 8, 3, 300), (3, 3, 1, 1, 1), (130, 1, 130, 5, 33),
                                                  (12, 3, 3, 2, 40), (256, 4, 256, 256, 9)])
def test_the_router_chooses_within_the_best_groups(E, top, groups, keep, N):
    g = torch.Generator().manual_seed(E)
    z = torch.randn((N, E + 2), generator=g) * 2
    s = torch.softmax(z[:, :E].double(), -1)
    want = P.choose_experts(s, top, groups, keep)
    choice, weight = ops().moe_route_groups(z.cuda(), E, top, softmax=True, groups=groups, keep=keep)
    assert torch.equal(choice.cpu().long(), want)                  # the largest first, as topk gives them
    assert float((weight.cpu().double() - torch.gather(s, 1, want)).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,E,top,F,W", [(3, 4, 2, 24, 48), (70, 8, 3, 64, 128), (1, 3, 1, 10, 36), (300, 6, 2, 96, 64)])
def test_experts_of_one_matrix_weighted_on_what_they_return(dtype, N, E, top, F, W):
    """Streamed (few pairs, float32 at any number) and grouped on the matrix cores, against the plain function."""
    g = torch.Generator().manual_seed(N + E)
    h = torch.randn((N, W), generator=g).to(dtype)
    up = (torch.randn((E, F, W), generator=g) * (1.5 / W ** 0.5)).to(dtype)
    down = (torch.randn((E, W, F), generator=g) / F ** 0.5).to(dtype)
    choice = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(N)]).int()
    weight = torch.rand((N, top), generator=g)
    want = torch.zeros((N, W), dtype=torch.float64)
    st = None if dtype == torch.float32 else dtype
    for n in range(N):
        for kk in range(top):
            e = int(choice[n, kk])
            tw = {"x.up": up[e].double(), "x.down": down[e].double()}
            want[n] += weight[n, kk].double() * P.dense_ffn(tw, "x", h[n:n + 1].double(), st)[0]
    got = ops().table_moe(h.cuda(), up.cuda(), down.cuda(), None, choice.cuda(), 1.0, out_scale=weight.cuda(), gated=False)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_embedding_hashes_pairs_across_steps(dtype):
    o = ops()
    g = torch.Generator().manual_seed(2)
    V, W, buckets = 29, 40, 7
    table, pairs = torch.randn((V, W), generator=g).to(dtype), torch.randn((buckets + 1, W), generator=g).to(dtype)
    seqs = {0: random_tokens(9, V, 1), 3: random_tokens(5, V, 2), 1: random_tokens(1, V, 3)}
    prev = torch.full((5,), 11, dtype=torch.int32, device="cuda")
    # step one: the first tokens of three requests in slots 0, 3, 1; step two: the rest of two of them
    for lens, first in (([4, 2, 1], [0, 0, 0]), ([5, 3], [4, 2])):
        slots = [0, 3, 1][:len(lens)]
        ids = [t for s, n, f in zip(slots, lens, first) for t in seqs[s][f:f + n]]
        b = batch_of(lens, slots, first, ids=ids)
        x, kept = o.hashed_pair_embedding(b, table.cuda(), pairs.cuda(), prev, 5, 3, keep=True)
        assert torch.equal(x, kept)
        at = 0
        for s, n, f in zip(slots, lens, first):
            rows = P.bigram_rows(seqs[s], buckets, 5, 3)[f:f + n]
            want = table[seqs[s][f:f + n]].double() + pairs[rows].double()
            assert float((x[at:at + n].double().cpu() - want).abs().max()) < 1e-6
            at += n
    assert prev.cpu().tolist() == [seqs[0][-1], seqs[1][-1], 11, seqs[3][-1], 11]


@pytest.mark.parametrize("dtype", DTYPES)
def test_small_elementwise_kernels(dtype):
    o = ops()
    g = torch.Generator().manual_seed(4)
    a, b = torch.randn((13, 20), generator=g), torch.randn((13, 12), generator=g)
    assert torch.equal(o.concat_rows(a.cuda(), b.cuda(), dtype).cpu(), torch.cat([a, b], 1).to(dtype))
    z = (torch.randn((13, 37), generator=g) * 2).to(dtype)
    close(o.relu_squared(z.cuda()[:, :33]), P.relu_squared(z[:, :33].double()), dtype)
    table = torch.randn((9, 30), generator=g).to(dtype)
    ids = torch.tensor(random_tokens(13, 9, 1), dtype=torch.int32)
    want = P.gelu_tanh(z[:, :6].double()) * table[ids.long()][:, 12:18].double()
    close(o.gate_table(z.cuda()[:, :6], ids.cuda(), table.cuda(), 12), want, dtype)


# ---------------------------------------------------------------- the engine against the plain implementation


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,index", [("A", 0), ("A", 1), ("A", 2), ("A", 3), ("M", 0), ("M", 1)])
def test_every_kind_of_layer_alone(tmp_path, which, index, dtype):
    from lmsf_amd.engine import StepEntry, load_engine_core
    cfg = single_layer(which, index, keep_loop=index % 2 == 1)
    folder, cfg, w = make_model(tmp_path, cfg, 3, decisive=dtype == "bfloat16")
    toks = random_tokens(90, cfg["vocab"], 11)
    core = load_engine_core(folder, dtype=dtype, block_size=8, num_pages=16, max_model_len=128, max_num_seqs=2)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in (37, 2, 30, 1, 1, 1, 18)])["a"]
    check(got, plain_logits(cfg, w, toks), dtype, (which, index), (cfg, w, toks))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "M"])
def test_four_ways_of_cutting_give_the_plain_logits(tmp_path, which, dtype):
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = make_model(tmp_path, which, 1, decisive=dtype == "bfloat16")
    lens = [150, 1, 37, 260, 5, 64]
    reqs = {"r%d" % i: random_tokens(n, cfg["vocab"], 30 + i) for i, n in enumerate(lens)}
    refs = {rid: plain_logits(cfg, w, toks) for rid, toks in reqs.items()}
    page = 16 if which == "M" else 8
    alone = -(-max(lens) // page) + 1
    for what, steps, pages in (("whole", trace_whole(reqs), alone),
                               ("bulk then single", trace_bulk_then_single(reqs, tail=20), alone),
                               ("portions", trace_portions(reqs, seed=3), alone),
                               ("mixed", trace_mixed(reqs, 512, seed=4), 512 // page)):
        core = load_engine_core(folder, dtype=dtype, block_size=page, num_pages=pages, max_model_len=pages * page,
                                max_num_seqs=4)
        got = replay_in_process(core.executor, steps)
        for rid in reqs:
            check(got[rid], refs[rid], dtype, (what, rid), (cfg, w, reqs[rid]))
        mgr = core.storage.manager
        mgr.check_invariants()
        assert all(mgr.num_free_pages(g) == pages for g in range(len(mgr.groups))) and mgr.num_free_state_slots() == 4
        del core


def far_token_model(n=200):
    """One layer of the delta rule whose memory holds one far token: the stream has an entry that only token X sets
    and one that every token sets alike; beta reads them, so that X writes with all its weight and the others hardly
    at all; the decays are close to 1. Returns the configuration, the weights and two sequences that differ in their
    first token (X or not)."""
    far = single_layer("C", 1)
    w = make_weights(far, 6)
    X = 0
    w["l0.mix.A_log"][:] = -6.0
    w["embed"][:, 0], w["embed"][:, 1] = 0.0, 2.0
    w["embed"][X, 0] = 4.0
    w["bigram"][:, :2] = 0.0
    w["l0.norm1"][:2] = 0.0
    w["l0.mix.b"][:] = 0.0
    w["l0.mix.b"][:, 1], w["l0.mix.b"][:, 0] = -6.0, 20.0
    w = {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}
    a = [X] + [1 + t % (far["vocab"] - 1) for t in random_tokens(n - 1, 1000, 13)]
    return far, w, a, [1] + a[1:]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_a_windows_edges_and_far_away_decide(tmp_path, dtype):
    """Peaked attention with a window: the plain implementation says which single tokens move the last logits (10
    back: yes; 11 back: no); the engine agrees on each sequence, in prompts and decoding. And the delta rule's memory
    with slow decays and a beta that lets one token write: the first token of 200 decides the last logits."""
    from lmsf_amd.engine import StepEntry, load_engine_core
    att = single_layer("A", 1)
    att["embedding"] = {"bigram": {"buckets": 5, "mul_prev": 0, "mul_cur": 3}}    # (a token's pair row: its own alone)
    folder, att, w = make_model(tmp_path, att, 5, spread=4.0, decisive=dtype == "bfloat16")
    size = att["layers"][0]["mixer"]["mask"]["size"]
    base = random_tokens(60, att["vocab"], 12)
    at_in, at_out = 59 - (size - 1), 59 - size
    ref = {"base": plain_logits(att, w, base)}

    def moved(at, v):
        return float((plain_logits(att, w, base[:at] + [v] + base[at + 1:])[-1] - ref["base"][-1]).abs().max())

    v = max((x for x in range(att["vocab"]) if x != base[at_in]), key=lambda x: moved(at_in, x))
    inside = base[:at_in] + [v] + base[at_in + 1:]
    outside = base[:at_out] + [v if v != base[at_out] else (v + 1) % att["vocab"]] + base[at_out + 1:]
    ref.update(inside=plain_logits(att, w, inside), outside=plain_logits(att, w, outside))
    assert float((ref["inside"][-1] - ref["base"][-1]).abs().max()) > 0.1 * float(ref["base"].double().std())
    assert float((ref["outside"][-1] - ref["base"][-1]).abs().max()) == 0.0
    for cuts in ([60], [45] + [1] * 15, [37, 2, 21]):
        core = load_engine_core(folder, dtype=dtype, block_size=4, num_pages=16, max_model_len=64, max_num_seqs=2)
        for k, t in (("base", base), ("inside", inside), ("outside", outside)):
            got = replay(core.executor, StepEntry, {k: t}, [[(k, c)] for c in cuts])[k]
            check(got, ref[k], dtype, (k, cuts), (att, w, t))
    far, w, a, b = far_token_model()
    folder, far, w = make_model(tmp_path, far, 6, weights=w)
    ra, rb = plain_logits(far, w, a), plain_logits(far, w, b)
    assert float((ra[-1] - rb[-1]).abs().max()) > 0.5 * float(ra.double().std())
    core = load_engine_core(folder, dtype=dtype, block_size=8, num_pages=4, max_model_len=208, max_num_seqs=1)
    for k, t, r in (("a", a, ra), ("b", b, rb)):
        got = replay(core.executor, StepEntry, {k: t}, [[(k, c)] for c in [130, 3, 50] + [1] * 17])[k]
        check(got, r, dtype, k, (far, w, t))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_graphs_equals_eager(tmp_path, dtype):
    from lmsf_amd.engine import StepEntry, load_engine_core
    folder, cfg, w = make_model(tmp_path, "A", 7, decisive=dtype == "bfloat16")
    reqs = {"a": random_tokens(140, cfg["vocab"], 1), "b": random_tokens(111, cfg["vocab"], 2)}
    steps = [[("a", 20), ("b", 3)]] + [[("a", 1), ("b", 1)]] * 100 + [[("a", 1)]] * 20 + [[("b", 1)]] * 8
    outs = []
    for eager in (True, False):
        core = load_engine_core(folder, dtype=dtype, block_size=8, num_pages=40, max_model_len=160, max_num_seqs=2,
                                enforce_eager=eager)
        outs.append(replay(core.executor, StepEntry, reqs, steps))
    for k, t in reqs.items():
        assert torch.equal(outs[0][k], outs[1][k]), k
        check(outs[1][k], plain_logits(cfg, w, t), dtype, k, (cfg, w, t))


def draw_config(seed):
    rng = random.Random(seed)
    pick = rng.choice

    def mlp():
        r = rng.random()
        if r < 0.2:
            return None
        if r < 0.5:
            return dense(pick([24, 100, 172]))
        per, count = pick([1, 2, 3, 4]), pick([1, 2, 3, 4])
        keep = pick(range(1, count + 1))
        top = pick([t for t in (1, 2, 3, 4) if t <= per * keep])
        return moe(per * count, top, pick([8, 20, 64]), groups=(count, keep) if count > 1 or rng.random() < 0.5 else None)

    W = pick([40, 72, 100, 136, 256])
    layers = []
    for i in range(pick([2, 3, 4, 5])):
        if rng.random() < 0.5:
            G = pick([1, 2, 3])
            d, dv = pick([8, 12, 20, 40, 64]), pick([8, 12, 24, 80])
            layers.append(attn(G * pick([1, 2, 3]), G, d, dv, pick([2, d // 2 // 2 * 2, d]), pick([1, 5, 16, 37, 64, 130, 500]),
                               scale=pick([None, 0.2]), softcap=pick([None, 4.0, 30.0]), base=pick([100.0, 10000.0, 5e5]),
                               mlp=mlp()))
        else:
            G = pick([1, 2, 3])
            layers.append(delta(G * pick([1, 2]), G, pick([8, 12, 20, 24, 64, 72]), pick([4, 8, 20, 33, 64, 100]),
                                pick([1, 2, 4, 5]), ranks=(pick([2, 8, 24]), pick([3, 8, 16])), mlp=mlp()))
    n = len(layers)
    loop = None
    if rng.random() < 0.75:
        a = pick(range(n))
        loop = (a, pick(range(a + 1, n + 1)), pick([1, 2, 3]))
    cfg = model(pick([41, 97, 256, 331]), W, layers, eps=pick([1e-5, 1e-6]),
                bigram=(pick([1, 13, 257]), pick([0, 1, 31, 1000003]), pick([1, 7, 65537])), side=pick([None, 4, 10, 32]),
                loop=loop)
    return cfg, pick([4, 8, 16, 32]), [pick([1, 2, 5, 17, 40, 77, 130, 200, 300]) for _ in range(5)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_a_configuration_drawn_at_random(tmp_path, seed, dtype):
    from lmsf_amd.engine import load_engine_core
    cfg, page, lens = draw_config(seed)
    folder, cfg, w = make_model(tmp_path, cfg, seed, decisive=dtype == "bfloat16")
    reqs = {"r%d" % i: random_tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(lens)}
    refs = {rid: plain_logits(cfg, w, toks) for rid, toks in reqs.items()}
    worst32 = 0.0
    if dtype == "float32":
        worst32 = max(rel_err(plain_logits(cfg, w, toks, dtype=torch.float32), refs[rid]) for rid, toks in reqs.items())
    alone = -(-max(lens) // page) + 1
    for what, steps, pages in (("whole", trace_whole(reqs), alone),
                               ("bulk then single", trace_bulk_then_single(reqs, tail=8), alone),
                               ("portions", trace_portions(reqs, seed=seed), alone),
                               ("mixed", trace_mixed(reqs, 512, seed=seed), 512 // page)):
        core = load_engine_core(folder, dtype=dtype, block_size=page, num_pages=pages, max_model_len=pages * page,
                                max_num_seqs=4)
        got = replay_in_process(core.executor, steps)
        for rid in reqs:
            assert torch.isfinite(got[rid]).all(), (what, rid, cfg)
            check(got[rid], refs[rid], dtype, (what, rid, cfg, page), (cfg, w, reqs[rid]), yardstick=worst32)
        core.storage.manager.check_invariants()
        assert core.storage.manager.num_free_state_slots() == 4
        del core


def test_greedy_generation_through_the_entry_point(tmp_path):
    from lmsf_amd.engine import LLM
    from lmsf_amd.sampling import SamplingParams
    folder, cfg, w = make_model(tmp_path, "A", 2)
    prompts = [random_tokens(n, cfg["vocab"], 40 + n) for n in (1, 9, 40)]
    llm = LLM(model=folder, dtype="float32", block_size=8, num_gpu_blocks_override=40, max_num_seqs=2,
              prefill_chunk_size=16, max_model_len=200)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert list(o.outputs[0].token_ids) == greedy(cfg, w, p, 6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_trace_runner_as_a_program(tmp_path, dtype):
    """bin/trace_run as a child process on a model folder: it picks the class by config.json, and a mixed schedule in a
    pool of 256 tokens with four state slots gives the plain logits."""
    folder, cfg, w = make_model(tmp_path, "A", 4, decisive=dtype == "bfloat16")
    lens = [90, 1, 37, 120, 5, 64]
    reqs = {"r%d" % i: random_tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate(lens)}
    steps = trace_mixed(reqs, 256, seed=5)
    got = replay_with_program(os.path.join(ROOT, "bin", "trace_run"), folder, dtype, steps, str(tmp_path / "out"), 256,
                              cfg["vocab"])
    for rid, toks in reqs.items():
        check(got[rid], plain_logits(cfg, w, toks), dtype, rid, (cfg, w, toks))


def test_the_command_line_generates(tmp_path):
    folder, cfg, w = make_model(tmp_path, "D", 3)
    prompt = random_tokens(11, cfg["vocab"], 9)
    proc = subprocess.run([os.path.join(ROOT, "bin", "lmsf_generate"), "--model", folder, "--dtype", "float32",
                           "--gpu-memory-utilization", "0.5", "--block-size", "8", "--max-model-len", "64",
                           "--prompt-ids", ",".join(map(str, prompt)), "--temperature", "0", "--max-tokens", "8",
                           "--ignore-eos"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [int(t) for t in proc.stdout.strip().splitlines()[0].split()] == greedy(cfg, w, prompt, 8)
