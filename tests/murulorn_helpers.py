"""Small Murulorn configurations and random weights by checkpoint name, made without the package's help, for the tests
that compare the engine with the plain implementation (plain_murulorn.py)."""
import json
import math
import os

import torch
from safetensors.torch import save_file

import plain_murulorn as P
from takosun_helpers import rel_err, replay, row_errs, within  # noqa: F401  (shared measures, re-exported)


def attn(heads, kv_heads, dim, vdim, rot, window, scale=None, softcap=None, base=10000.0, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5,
         "rot": {"base": base, "dims": rot}, "mask": {"size": window}}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def delta(heads, kv_heads, dim, vdim, conv, ranks=(6, 10), mlp=None):
    """``ranks``: the rows of a1 and g1 (no key of the configuration: the tensors' shapes give them)."""
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                               "conv": conv, "_ranks": list(ranks)}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def model(vocab, width, layers, eps=1e-5, bigram=(37, 11, 5), side=None, loop=None):
    cfg = {"architecture": "Murulorn", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}, "layers": layers}
    if side:
        cfg["token_side"] = {"dim": side}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# Sizes differ between the configurations and inside each: one to six heads with one to three heads of keys, values
# wider and narrower than keys, windows of 1 to 50 positions that are no multiples of a page, rotation of a whole head
# and of part of it, with and without a soft cap, two to five taps, one to three of three to eight experts in one to
# four groups, layers without a feed-forward, a loop in the middle, over everything, of one pass and none, with and
# without the tokens' side inputs, a model without attention and one without the delta rule.
CONFIGS = {
    "A": model(61, 48, [
        delta(2, 1, 8, 12, 3, ranks=(5, 7), mlp=dense(40)),
        attn(4, 2, 12, 8, 6, 11, scale=0.3, softcap=5.0, mlp=moe(6, 2, 16, groups=(3, 2))),
        delta(3, 3, 16, 4, 2, ranks=(8, 3), mlp=moe(4, 1, 12)),
        attn(2, 1, 8, 20, 8, 40, base=300.0),
    ], side=6, loop=(1, 3, 2)),
    "B": model(77, 64, [      # pages only: no delta rule, no loop, no side input
        attn(1, 1, 24, 24, 24, 1, mlp=dense(72)),
        attn(6, 3, 4, 8, 2, 19, softcap=50.0, base=50.0, mlp=moe(3, 3, 20)),
        attn(5, 5, 8, 4, 4, 7, scale=0.5, softcap=2.0),
    ], eps=1e-6, bigram=(1, 0, 1)),
    "C": model(40, 32, [      # state only: no pages at all; everything loops
        delta(2, 2, 12, 12, 4, ranks=(4, 4), mlp=moe(8, 3, 16, groups=(4, 2))),
        delta(1, 1, 20, 6, 5, ranks=(3, 9), mlp=dense(24)),
    ], side=3, loop=(0, 2, 3), bigram=(53, 1, 1)),
    "D": model(53, 40, [      # a loop of one pass at the end
        attn(2, 2, 20, 16, 20, 13, mlp=moe(4, 2, 8, groups=(2, 1))),
        delta(4, 2, 8, 8, 2, ranks=(2, 2)),
    ], side=8, loop=(1, 2, 1), bigram=(7, 3, 2)),
    # sizes at which the matrix-core forms of the kernels run (GPU tests)
    "M": model(300, 192, [
        attn(4, 2, 64, 64, 32, 50, scale=0.125, softcap=20.0, base=1e5, mlp=dense(512)),
        delta(4, 2, 64, 128, 4, ranks=(16, 24), mlp=moe(8, 2, 128, groups=(4, 2))),
        attn(2, 1, 128, 96, 128, 90, softcap=30.0, mlp=moe(8, 2, 128)),
        delta(2, 2, 128, 64, 3, ranks=(8, 8), mlp=dense(384)),
    ], side=16, loop=(1, 3, 2), bigram=(1009, 31, 7)),
}


def make_weights(cfg, seed, spread=1.0, decisive=False):
    """Matrices N(0, 1 / inputs) (the norms of queries ``spread`` times larger, so that attention is peaked for
    spread > 1); norm weights of the layers around 0 (they act as 1 + w), the others around 1; routers wide enough
    that the scores differ.

    ``decisive``: no choice of experts is a close call, so that rounding cannot flip one (a flipped choice moves a
    row, and every later row, by far more than rounding; bfloat16 runs are compared under such weights, float32 runs
    under the random routers). The last E entries of the stream (E: the most experts of a layer) hold a code of the
    token id, distinct levels in an order that turns with the id; no sublayer, side input or pair row writes to them
    and the matrix that begins a pass hands them on as they are; expert e's router row reads entry e with a large
    factor beside small random entries."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    w = {}

    def mat(name, rows, cols, s=1.0):
        w[name] = torch.randn((rows, cols), generator=g) * (s / math.sqrt(cols))

    def around(name, n, centre=1.0, dev=0.2):
        w[name] = centre + dev * torch.randn((n,), generator=g)

    w["embed"] = torch.randn((V, W), generator=g)
    w["bigram"] = torch.randn((cfg["embedding"]["bigram"]["buckets"] + 1, W), generator=g) * 0.7
    L = len(cfg["layers"])
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        w["side.embed"] = torch.randn((V, L * side), generator=g)
    if cfg.get("loop"):
        mat("loop.in", W, 2 * W, 1.2)
    for i, lay in enumerate(cfg["layers"]):
        p, m, q = "l%d" % i, lay["mixer"], "l%d.mix" % i
        around(p + ".norm1", W, 0.0), around(p + ".norm1b", W, 0.0)
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if lay["type"] == "attention":
            mat(q + ".q", H * d, W), mat(q + ".k", G * d, W), mat(q + ".v", G * dv, W), mat(q + ".g", H, W)
            around(q + ".q.norm", H * d, spread), around(q + ".k.norm", G * d)
            mat(q + ".o", W, H * dv)
        else:
            ra, rg = m["_ranks"]
            taps = m["conv"]
            mat(q + ".q", G * d, W, 1.5), mat(q + ".k", G * d, W, 1.5), mat(q + ".v", H * dv, W, 1.5)
            for x, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
                w["%s.%s.conv" % (q, x)] = torch.randn((n, taps), generator=g) * 0.6
            mat(q + ".b", H, W), mat(q + ".a1", ra, W), mat(q + ".a2", H * d, ra, 1.5)
            w[q + ".dt_bias"] = torch.randn((H * d,), generator=g)
            w[q + ".A_log"] = torch.rand((H,), generator=g) * 2.0 - 1.5
            mat(q + ".g1", rg, W), mat(q + ".g2", H * dv, rg, 1.5)
            around(q + ".norm", dv)
            mat(q + ".o", W, H * dv)
        if side:
            mat(p + ".side.gate", side, W), mat(p + ".side.proj", W, side)
            around(p + ".side.norm", W, 0.5, 0.1)
        mlp = lay["mlp"]
        if mlp is None:
            continue
        around(p + ".norm2", W, 0.0), around(p + ".norm2b", W, 0.0)
        if mlp["kind"] == "dense":
            mat(p + ".mlp.up", mlp["ff"], W, 1.5), mat(p + ".mlp.down", W, mlp["ff"])
        else:
            F = mlp["expert"]["ff"]
            mat(p + ".mlp.router", mlp["router"]["experts"], W, 2.0)
            for e in range(mlp["router"]["experts"]):
                x = "%s.mlp.e%d" % (p, e)
                mat(x + ".up", F, W, 1.5), mat(x + ".down", W, F)
    around("final.norm", W, 0.0)
    most = max([lay["mlp"]["router"]["experts"] for lay in cfg["layers"]
                if lay["mlp"] is not None and lay["mlp"]["kind"] == "moe"], default=0)
    if decisive and most:
        code = list(range(W - most, W))
        levels = torch.linspace(-1.5, 1.5, most) if most > 1 else torch.zeros(1)
        for t in range(V):
            w["embed"][t, code] = torch.roll(levels, t % most)
        w["bigram"][:, code] = 0.0
        for name in list(w):
            if name.endswith(".o") or name.endswith(".down") or name.endswith(".side.proj"):
                w[name][code, :] = 0.0
            elif name.endswith(".router"):
                w[name] *= 0.1
                for e in range(w[name].shape[0]):
                    w[name][e, code[e]] += 10.0
            elif name.endswith(".norm2"):
                w[name][code] = 0.0
            elif name == "loop.in":
                w[name][code, :] = 0.0
                w[name][:, code] = 0.0
                w[name][:, [W + c for c in code]] = 0.0
                for c in code:
                    w[name][c, c] = 1.0
    # the values a bfloat16 checkpoint holds, so that every run sees the same numbers
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}


def public(cfg):
    """The configuration as config.json holds it: without the helpers' own keys."""
    out = json.loads(json.dumps(cfg))
    for lay in out["layers"]:
        for k in [k for k in lay["mixer"] if k.startswith("_")]:
            del lay["mixer"][k]
    return out


def write_model(folder, cfg, weights):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(public(cfg), f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def make_model(tmp_path, which, seed=0, spread=1.0, weights=None, decisive=False):
    cfg = CONFIGS[which] if isinstance(which, str) else which
    weights = weights if weights is not None else make_weights(cfg, seed, spread, decisive)
    tag = which if isinstance(which, str) else "custom"
    folder = write_model(os.path.join(str(tmp_path), "murulorn_%s_%d_%g_%d" % (tag, seed, spread, decisive)), cfg, weights)
    return folder, cfg, weights


def plain_logits(cfg, weights, tokens, dtype=torch.float64, storage=None):
    return P.forward(cfg, weights, tokens, dtype=dtype, storage=storage).to(torch.float32)


def greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(plain_logits(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]


def bfloat16_limits(cfg, weights, tokens, ref, draws=3):
    """What rounding to bfloat16 may cost at every position: three times what it costs the plain implementation when
    it rounds what an engine may keep in 16 bits, the largest of ``draws`` draws of the rounding errors, but no less
    than three times the median of the first draw over the positions."""
    e = row_errs(plain_logits(cfg, weights, tokens, dtype=torch.float32, storage=torch.bfloat16), ref)
    worst = torch.maximum(e, e.median())
    for i in range(1, draws):
        gen = torch.Generator().manual_seed(1000 + i)
        worst = torch.maximum(worst, row_errs(plain_logits(cfg, weights, tokens, dtype=torch.float32,
                                                           storage=(torch.bfloat16, gen)), ref))
    return 3.0 * worst


def single_layer(which, index, vocab=47, keep_loop=False):
    """The configuration of one layer of ``which`` alone (a mechanism on its own), without loop unless asked."""
    cfg = CONFIGS[which]
    out = dict(cfg)
    out.update(vocab=vocab, layers=[json.loads(json.dumps(cfg["layers"][index]))])
    out.pop("loop", None)
    if keep_loop:
        out["loop"] = {"start": 0, "stop": 1, "times": 2}
    return out
