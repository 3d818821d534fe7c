"""Zevetar on the GPU: the new kernels alone against the plain implementation's function of the same mechanism, every
kind of layer alone and the whole model through the engine's step function in float32 and bfloat16 under the ways of
cutting a request into steps, keys at a window's edges and far away made to decide the logits, pages and state slots
used again, long decoding from graphs, configurations drawn at random, and generation through the entry point."""
import math
import random
from types import SimpleNamespace

import pytest
import torch

import plain_zevetar as P
from helpers import random_tokens, replay_in_process, trace_bulk_then_single, trace_mixed, trace_portions, trace_whole
from zevetar_helpers import (YARN, bfloat16_limits, dense, latent, make_model, make_weights, model, moe, plain_logits,
                             rel_err, replay, ret, single_layer, within)

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL_F32 = 3e-5


def ops():
    from lmsf_amd.ops import get_ops
    return get_ops()


def close(got, ref, dtype, scale=1.0):
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    err = float((got.double().cpu() - ref.double().cpu()).abs().max())
    assert err <= tol * max(scale, float(ref.double().abs().max())), (err, float(ref.double().abs().max()))


def check(got, ref, dtype, what, model_):
    """float32: three times what float32 rounding costs the plain implementation itself, where that is more than
    TOL_F32; bfloat16: per position three times what rounding costs the plain implementation when it rounds what an
    engine may keep in 16 bits."""
    cfg, w, toks = model_
    if dtype == "float32":
        tol = max(TOL_F32, 3 * rel_err(plain_logits(cfg, w, toks, dtype=torch.float32), ref))
        assert rel_err(got, ref) < tol, (what, rel_err(got, ref), tol)
    else:
        ok, worst = within(got, ref, bfloat16_limits(cfg, w, toks, ref))
        assert ok, (what, worst)


def batch_of(lens, slots, first_pos=None, dev="cuda"):
    """What the state-carrying kernels read of a step: segments of ``lens`` tokens in state slots ``slots``."""
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    first_pos = first_pos or [0] * len(lens)
    pos = [p0 + i for p0, n in zip(first_pos, lens) for i in range(n)]
    seg = [s for s, n in enumerate(lens) for _ in range(n)]
    i32 = dict(dtype=torch.int32, device=dev)
    return SimpleNamespace(n_segments=len(lens), seg_starts=torch.tensor(starts, **i32), state_slots=torch.tensor(slots, **i32),
                           seg_of_token=torch.tensor(seg, **i32), positions=torch.tensor(pos, **i32),
                           host_seg_lens=list(lens), all_single=all(n == 1 for n in lens), replayed=False, aux={})


# ---------------------------------------------------------------- kernels alone


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,dv,rot,lens", [(3, 8, 20, 4, [5, 1, 17]), (2, 64, 96, 64, [300, 2, 70]), (1, 24, 8, 0, [1, 1, 1]),
                                              (4, 128, 40, 32, [130, 64]), (2, 20, 33, 20, [16, 47, 200]),
                                              (2, 256, 16, 0, [50, 2]), (1, 320, 24, 64, [40, 5])])
def test_retention_in_all_its_forms_against_the_recurrence(dtype, H, d, dv, rot, lens):
    """Token by token, chunks one after the other and chunks side by side, each segment continued from a state that
    an earlier step left, against the plain recurrence in float64. Heads of up to 256 entries take the matrix-core
    form of the chunks (64, 32 or 16 tokens a chunk), wider ones the scalar form."""
    o = ops()
    g = torch.Generator().manual_seed(H * 100 + d)
    decay = [1.0, 0.9, 0.5, 0.999][:H]
    slots = [2, 0, 3][:len(lens)]
    first = [7, 0, 40][:len(lens)]
    N = sum(lens)
    p = (torch.randn((N, 2 * H * d + 2 * H * dv), generator=g) * 0.7).to(dtype)
    state0 = torch.randn((5, H * d * dv + 3), generator=g)
    state0[0] = 0
    table = None
    if rot:
        inv = 50.0 ** (-torch.arange(rot // 2, dtype=torch.float32) * 2 / rot)
        ang = torch.arange(400, dtype=torch.float32)[:, None] * inv[None, :]
        table = torch.cat([torch.cos(ang), torch.sin(ang)], 1).contiguous()
    # the plain recurrence
    pd = p.double()
    want = torch.empty((N, H * dv), dtype=torch.float64)
    st = state0.double().clone()
    at = 0
    for n, slot, p0 in zip(lens, slots, first):
        S = st[slot, :H * d * dv].reshape(H, d, dv)
        for t in range(at, at + n):
            q, k = pd[t, :H * d].reshape(1, H, d), pd[t, H * d:2 * H * d].reshape(1, H, d)
            if rot:
                pos = torch.tensor([p0 + t - at])
                q, k = P.rotate(q, pos, rot, 50.0, None, False), P.rotate(k, pos, rot, 50.0, None, False)
            v = pd[t, 2 * H * d:2 * H * d + H * dv].reshape(H, dv)
            S = torch.tensor(decay, dtype=torch.float64)[:, None, None] * S + (k[0] * d ** -0.5)[:, :, None] * v[:, None, :]
            oo = torch.einsum("hde,hd->he", S, q[0])
            oo = P.rms_norm(oo, None, 1e-5).reshape(-1)
            want[t] = oo * P.silu(pd[t, 2 * H * d + H * dv:])
        st[slot, :H * d * dv] = S.reshape(-1)
        at += n
    dec = torch.tensor(decay + [math.log(x) for x in decay], dtype=torch.float32, device="cuda")
    state = state0.cuda()
    pc = p.cuda()
    got = o.retention(pc[:, :H * d], pc[:, H * d:2 * H * d], pc[:, 2 * H * d:2 * H * d + H * dv], dec,
                      pc[:, 2 * H * d + H * dv:], state, batch_of(lens, slots, first), H, d, dv, d ** -0.5, 1e-5,
                      table=table.cuda() if table is not None else None)
    close(got, want, dtype, scale=1.0)
    assert float((state.cpu().double() - st).abs().max()) <= 3e-5 * max(1.0, float(st.abs().max()))
    assert torch.equal(state.cpu()[:, H * d * dv:], state0[:, H * d * dv:])        # what lies behind is not touched


@pytest.mark.parametrize("E,top,N", [(5, 2, 7), (64, 6, 300), (3, 3, 1), (130, 1, 33)])
def test_the_router_takes_the_largest_scores_first(E, top, N):
    g = torch.Generator().manual_seed(E)
    z = torch.randn((N, E + 1), generator=g) * 2
    z[0, :] = 0.25                                     # equal scores: the lower index first
    for renorm in (False, True):
        choice, weight, gate = ops().moe_route(z.cuda(), E, top, renorm=renorm, extra=E)
        s = torch.sigmoid(z[:, :E])
        order = torch.argsort(-z[:, :E], dim=-1, stable=True)[:, :top]
        assert torch.equal(choice.cpu().long(), order)
        w = torch.gather(s, 1, order)
        w = w / w.sum(-1, keepdim=True) if renorm else w
        assert float((weight.cpu() - w).abs().max()) < 1e-6
        assert float((gate.cpu() - torch.sigmoid(z[:, E])).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,E,top,F,W", [(3, 5, 2, 24, 48), (70, 4, 3, 20, 40), (200, 8, 2, 128, 256), (1, 3, 1, 12, 32)])
def test_experts_with_a_weight_on_their_input_and_a_gated_base(dtype, N, E, top, F, W):
    """Streamed and grouped forms: out = gate * base + sum_k y_e(s_k h) against the plain gated feed-forward."""
    g = torch.Generator().manual_seed(N + E)
    h = (torch.randn((N, W), generator=g)).to(dtype)
    wgu = (torch.randn((E, 2 * F, W), generator=g) / math.sqrt(W)).to(dtype)
    wd = (torch.randn((E, W, F), generator=g) / math.sqrt(F)).to(dtype)
    base = torch.randn((N, W), generator=g).to(dtype)
    choice = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(N)]).to(torch.int32)
    scale = torch.rand((N, top), generator=g) + 0.1
    gate = torch.rand((N,), generator=g)
    got = ops().table_moe(h.cuda(), wgu.cuda(), wd.cuda(), None, choice.cuda(), 1.0, base=base.cuda(),
                          pair_scale=scale.cuda(), base_scale=gate.cuda())
    want = gate[:, None].double() * base.double()
    for n in range(N):
        for k in range(top):
            e = int(choice[n, k])
            x = scale[n, k].double() * h[n].double()
            gu = wgu[e].double() @ x
            want[n] += wd[e].double() @ (P.silu(gu[:F]) * gu[F:])
    close(got, want, dtype, scale=1.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,W,two,normed", [(5, 48, True, True), (300, 256, True, True), (3, 1000, False, True), (17, 40, True, False)])
def test_two_scaled_branches_join_the_stream_and_the_next_norm(dtype, N, W, two, normed):
    g = torch.Generator().manual_seed(W)
    a, b = torch.randn((N, W), generator=g).to(dtype), torch.randn((N, W), generator=g).to(dtype)
    sa, sb, wn = torch.rand(W, generator=g), torch.rand(W, generator=g), torch.rand(W, generator=g) + 0.5
    x = torch.randn((N, W), generator=g)
    stream = x.cuda()
    out = ops().scale_add_norm(a.cuda(), sa.cuda(), b.cuda() if two else None, sb.cuda() if two else None, stream,
                               weight=wn.cuda() if normed else None, eps=1e-6)
    want = x.double() + sa.double() * a.double() + (sb.double() * b.double() if two else 0)
    assert float((stream.cpu().double() - want).abs().max()) < 1e-5
    if normed:
        close(out, P.rms_norm(want, wn.double(), 1e-6), dtype)
    else:
        assert out is None


def test_logits_scaled_and_capped():
    x = torch.randn((7, 333)) * 40
    for scale, cap in ((0.5, 30.0), (2.0, 0.0)):
        got = ops().logit_cap(x.clone().cuda(), scale, cap).cpu()
        want = cap * torch.tanh(x.double() * scale / cap) if cap else x.double() * scale
        assert float((got.double() - want).abs().max()) < 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,H,O,K", [(5, 3, 12, 24), (100, 4, 96, 128), (9, 2, 20, 32)])
def test_per_head_products_with_a_gate_for_every_output(dtype, N, H, O, K):
    g = torch.Generator().manual_seed(O)
    x = torch.randn((N, H * K), generator=g).to(dtype)
    w = (torch.randn((H, O, K), generator=g) / math.sqrt(K)).to(dtype)
    gate = torch.randn((N, H * O + 3), generator=g).to(dtype)
    out = torch.empty((N, H * O), dtype=dtype, device="cuda")
    ops().head_linear(x.cuda(), K, w.cuda(), out, O, gate=gate.cuda(), gate_wide=True)
    want = torch.einsum("nhk,hok->nho", x.double().reshape(N, H, K), w.double()).reshape(N, H * O) \
        * torch.sigmoid(gate[:, :H * O].double())
    close(out, want, dtype)


@pytest.mark.parametrize("d,ps,ctx,n_query", [(64, 16, 2, 1), (64, 16, 2, 2), (160, 8, 41, 1), (160, 8, 41, 41),
                                              (256, 4, 300, 1), (128, 16, 700, 130), (48, 32, 90, 3), (96, 4, 50, 50)])
def test_softmax_weights_in_float32_into_the_product_with_the_values(d, ps, ctx, n_query):
    """Values of +1 and -1 in turn under nearly equal weights: the result is a small difference of large sums, and what
    rounding the weights to bfloat16 costs (2^-9 of a weight) stands out against what rounding the result costs (2^-9
    of the result). With ``weights_f32`` every entry is within the result's own rounding of the float64 value; without
    it, it is not (which says that the case can tell)."""
    g = torch.Generator().manual_seed(d + ctx)
    nh, nkv = 8, 1
    pages = -(-ctx // ps)
    k = (torch.randn(pages, nkv, ps, d, generator=g) * 0.3).to(torch.bfloat16)
    sign = torch.tensor([1.0 if j % 2 == 0 else -1.0 for j in range(pages * ps)]).reshape(pages, 1, 1, ps)
    v = sign.expand(pages, nkv, d, ps).contiguous().to(torch.bfloat16)
    q = (torch.randn(n_query, nh * d, generator=g) * 0.05).to(torch.bfloat16)
    pos = torch.arange(ctx - n_query, ctx, dtype=torch.int32)
    seg = torch.zeros(n_query, dtype=torch.int32)
    bt = torch.arange(pages, dtype=torch.int32).reshape(1, pages)
    scale = d ** -0.5
    keys = k.double().permute(1, 0, 2, 3).reshape(nkv, pages * ps, d)[0]                     # [keys, d]
    want = torch.empty(n_query, nh, dtype=torch.float64)
    for i in range(n_query):
        n = int(pos[i]) + 1
        sc = (q[i].double().reshape(nh, d) @ keys[:n].T) * scale
        want[i] = (torch.softmax(sc, -1) * sign.reshape(-1)[:n].double()).sum(-1)
    errs = {}
    for exact in (True, False):
        got = ops().paged_attention(q.cuda(), k.cuda(), v.cuda(), bt.cuda(), seg.cuda(), pos.cuda(), nh, nkv, d, scale, 0,
                                    kernel="mfma", weights_f32=exact).cpu().double().reshape(n_query, nh, d)
        assert float((got - got[:, :, :1]).abs().max()) == 0.0           # every column of V is the same
        errs[exact] = (got[:, :, 0] - want).abs()
    bound = 2.0 ** -8 * want.abs() + 3e-6
    assert bool((errs[True] <= bound).all()), float((errs[True] / bound).max())
    assert float((errs[False] / bound).max()) > 3.0


# ---------------------------------------------------------------- through the engine


LAYERS_ALONE = [("A", 0), ("A", 1), ("A", 2), ("A", 3), ("B", 0), ("B", 1), ("B", 3), ("M", 1), ("M", 2), ("M", 3)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,index", LAYERS_ALONE)
def test_every_kind_of_layer_alone(tmp_path, which, index, dtype):
    from lmsf_amd.engine import StepEntry, load_engine_core
    cfg = single_layer(which, index)
    folder, cfg, w = make_model(tmp_path, cfg, 3, decisive=dtype == "bfloat16")
    toks = random_tokens(70, cfg["vocab"], 5)
    core = load_engine_core(folder, dtype=dtype, block_size=8, num_pages=12, max_model_len=96, max_num_seqs=2)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in (33, 2, 19, 1, 1, 1, 13)])["a"]
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_a_windows_edges_and_far_away_decide(tmp_path, dtype):
    """Peaked attention with a window and a retention head that forgets nothing: the plain implementation says which
    single tokens move the last logits (10 back: yes; 11 back, through attention alone: no; the first of 200, through
    a retention layer whose weights make that one score stand out: yes); the engine agrees on each sequence, in prompts and decoding."""
    from lmsf_amd.engine import StepEntry, load_engine_core
    att = single_layer("A", 0)
    folder, att, w = make_model(tmp_path, att, 5, spread=4.0)
    size = att["layers"][0]["mixer"]["mask"]["size"]
    base = random_tokens(60, att["vocab"], 12)
    at_in, at_out = 59 - (size - 1), 59 - size
    ref = {"base": plain_logits(att, w, base)}

    def moved(at, v):
        return float((plain_logits(att, w, base[:at] + [v] + base[at + 1:])[-1] - ref["base"][-1]).abs().max())

    # (peaked attention looks at few keys: of all tokens that could stand at the window's first place, take the one
    # that the last query looks at most)
    v = max((x for x in range(att["vocab"]) if x != base[at_in]), key=lambda x: moved(at_in, x))
    inside = base[:at_in] + [v] + base[at_in + 1:]
    outside = base[:at_out] + [v if v != base[at_out] else (v + 1) % att["vocab"]] + base[at_out + 1:]
    ref.update(inside=plain_logits(att, w, inside), outside=plain_logits(att, w, outside))
    assert float((ref["inside"][-1] - ref["base"][-1]).abs().max()) > 0.2 * float(ref["base"].double().std())
    assert float((ref["outside"][-1] - ref["base"][-1]).abs().max()) == 0.0
    for cuts in ([60], [45] + [1] * 15, [37, 2, 21]):
        core = load_engine_core(folder, dtype=dtype, block_size=4, num_pages=16, max_model_len=64, max_num_seqs=2)
        for k, t in (("base", base), ("inside", inside), ("outside", outside)):
            got = replay(core.executor, StepEntry, {k: t}, [[(k, c)] for c in cuts])[k]
            check(got, ref[k], dtype, (k, cuts), (att, w, t))
    # one key 199 tokens back among keys of equal weight: tokens X and Y get an entry of the stream each that no other
    # token has; the keys read X's entry and the queries Y's along one direction u, so that Y's query and X's key
    # give a score far above all others
    far = single_layer("B", 0)
    w = make_weights(far, 6)
    X, Y = 0, 1
    u = torch.randn(w["l0.mix.k"].shape[0], generator=torch.Generator().manual_seed(1))
    w["embed"][:, :2] = 0.0
    w["embed"][X], w["embed"][Y] = 0.0, 0.0
    w["embed"][X, 0], w["embed"][Y, 1] = 1.0, 1.0
    w["l0.mix.k"][:, 0] = w["l0.mix.q"][:, 1] = 4.0 * u / u.norm()
    w = {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}
    folder, far, w = make_model(tmp_path, far, 6, weights=w)
    a = [X] + [2 + t % (far["vocab"] - 2) for t in random_tokens(198, 1000, 13)] + [Y]
    b = [2] + a[1:]
    ra, rb = plain_logits(far, w, a), plain_logits(far, w, b)
    assert float((ra[-1] - rb[-1]).abs().max()) > 0.2 * float(ra.double().std())
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

    def mlp(W):
        r = rng.random()
        if r < 0.25:
            return None
        if r < 0.55:
            return dense(pick([24, 100, 172]))
        e = pick([2, 3, 7, 16])
        return moe(e, pick([t for t in (1, 2, 3, 4) if t <= e]), pick([8, 20, 64]), shared=pick([None, 12, 48]))

    W = pick([40, 72, 100, 136, 256])
    layers, owners = [], []
    for i in range(pick([2, 3, 4, 5])):
        if rng.random() < 0.6:
            window = pick([None, 1, 5, 16, 37, 64, 130])
            if owners and rng.random() < 0.4:
                j = pick(owners)
                m = layers[j]["mixer"]
                layers.append(latent(pick([1, 2, 3, 6]), pick([8, 12, 20, 40, 64]), m["rot_dim"], pick([8, 12, 24, 80]),
                                     m["kv_rank"], pick([8, 20, 48]), window=window, base=m["rot"]["base"],
                                     scaling=m["rot"].get("scaling"), scale=pick([None, 0.2]), kv_from=j, mlp=mlp(W)))
            else:
                owners.append(i)
                layers.append(latent(pick([1, 2, 3, 6]), pick([8, 12, 20, 40, 64]), pick([2, 4, 8, 16, 32]),
                                     pick([8, 12, 24, 80]), pick([8, 20, 44, 96, 300]), pick([8, 20, 48]), window=window,
                                     base=pick([100.0, 10000.0, 5e5]), scaling=pick([None, YARN]), scale=pick([None, 0.2]),
                                     mlp=mlp(W)))
        else:
            H, d = pick([1, 2, 3, 5]), pick([8, 12, 20, 24, 64, 72])
            layers.append(ret(H, d, pick([4, 8, 20, 33, 64, 100]), [pick([1.0, 0.999, 0.97, 0.9, 0.5, 0.1]) for _ in range(H)],
                              rot_dims=pick([None, 2, d // 2 // 2 * 2, d // 2 * 2]), base=pick([100.0, 1e6]), mlp=mlp(W)))
    cfg = model(pick([41, 97, 256, 331]), W, layers, eps=pick([1e-5, 1e-6]), emb=pick([1.0, 6.0]),
                logit_scale=pick([1.0, 0.3]), cap=pick([None, 8.0, 30.0]))
    return cfg, pick([4, 8, 16, 32]), [pick([1, 2, 5, 17, 40, 77, 130, 200, 300]) for _ in range(5)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_a_configuration_drawn_at_random(tmp_path, seed, dtype):
    from lmsf_amd.engine import load_engine_core
    cfg, page, lens = draw_config(seed)
    folder, cfg, w = make_model(tmp_path, cfg, seed, decisive=dtype == "bfloat16")
    reqs = {"r%d" % i: random_tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(lens)}
    refs = {rid: plain_logits(cfg, w, toks) for rid, toks in reqs.items()}
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
            check(got[rid], refs[rid], dtype, (what, rid, cfg, page), (cfg, w, reqs[rid]))
        core.storage.manager.check_invariants()
        assert core.storage.manager.num_free_state_slots() == 4
        del core


def test_greedy_generation_through_the_entry_point(tmp_path):
    from lmsf_amd.engine import LLM
    from lmsf_amd.sampling import SamplingParams
    folder, cfg, w = make_model(tmp_path, "B", 2)
    prompts = [random_tokens(n, cfg["vocab"], 40 + n) for n in (1, 9, 40)]
    llm = LLM(model=folder, dtype="float32", block_size=8, num_gpu_blocks_override=40, max_num_seqs=2,
              prefill_chunk_size=16, max_model_len=200)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert list(o.outputs[0].token_ids) == P.greedy(cfg, w, p, 6)
