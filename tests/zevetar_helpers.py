"""Small Zevetar configurations and random weights by checkpoint name, made without the package's help, for the tests
that compare the engine with the plain implementation (plain_zevetar.py)."""
import json
import math
import os

import torch
from safetensors.torch import save_file

import plain_zevetar as P
from takosun_helpers import rel_err, replay, row_errs, within  # noqa: F401  (shared measures, re-exported)

YARN = {"factor": 4.0, "original": 24, "fast": 8.0, "slow": 0.5}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, window=None, base=10000.0, scaling=None, scale=None, kv_from=None,
           mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale or (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim}}
    if scaling:
        m["rot"]["scaling"] = scaling
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def ret(heads, dim, vdim, decay, rot_dims=None, base=10000.0, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "retention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def model(vocab, width, layers, eps=1e-5, emb=1.0, logit_scale=1.0, cap=None):
    cfg = {"architecture": "Zevetar", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": emb}, "logit_scale": logit_scale, "layers": layers}
    if cap:
        cfg["logit_softcap"] = cap
    return cfg


# Sizes differ between the configurations and inside each: one to five heads, values wider and narrower than keys,
# windows of 1 to 40 positions that are no multiples of a page (and a layer that sees everything), a reader whose
# window is wider than its latent's owner's, one to three of three to six experts with and without a shared one, layers
# without a feed-forward, decays of 1 and far below, rotation of a whole head, of part of it and none, with and
# without YaRN, a model without attention and one without retention, no soft cap and scales of 1.
CONFIGS = {
    "A": model(61, 48, [
        latent(3, 16, 8, 12, 24, 20, window=11, scaling=YARN, mlp=dense(40)),
        latent(3, 16, 8, 12, 24, 20, window=19, scaling=YARN, kv_from=0, mlp=moe(5, 2, 24, shared=16)),
        ret(3, 8, 20, [0.9, 0.5, 1.0], rot_dims=4, mlp=moe(3, 1, 12)),
        latent(2, 8, 4, 24, 12, 16, base=300.0),
    ], emb=3.0, logit_scale=0.5, cap=12.0),
    "B": model(77, 64, [
        ret(1, 24, 8, [1.0]),
        latent(1, 12, 12, 20, 20, 8, window=1, mlp=dense(72)),
        ret(4, 16, 40, [0.99, 0.97, 0.8, 0.3], rot_dims=16, base=50.0, mlp=dense(32)),
        latent(5, 4, 8, 8, 8, 24, window=40, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0},
               mlp=moe(4, 3, 20, shared=36)),
        latent(5, 4, 8, 8, 8, 24, window=7, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}, kv_from=3),
    ], eps=1e-6, emb=1.0, logit_scale=2.0, cap=50.0),
    "C": model(40, 32, [      # state only: no pages at all
        ret(2, 12, 12, [0.95, 0.6], rot_dims=12, mlp=moe(6, 2, 16, shared=8)),
        ret(2, 20, 4, [0.999, 0.9], mlp=dense(24)),
    ], emb=5.0),
    "D": model(53, 40, [      # pages only: no state
        latent(2, 20, 4, 16, 28, 12, window=13, mlp=moe(3, 3, 8)),
        latent(4, 8, 8, 8, 8, 8, mlp=None),
    ], logit_scale=0.25, cap=3.0),
    # sizes at which the matrix-core forms of the kernels run (GPU tests)
    "M": model(300, 256, [
        latent(4, 64, 32, 96, 96, 64, window=50, base=1e5, scaling={"factor": 2.0, "original": 64, "fast": 16.0, "slow": 1.0},
               mlp=dense(512)),
        latent(4, 64, 32, 96, 96, 64, window=90, base=1e5, scaling={"factor": 2.0, "original": 64, "fast": 16.0, "slow": 1.0},
               kv_from=0, mlp=moe(8, 2, 128, shared=256)),
        ret(4, 64, 128, [0.98, 0.9, 0.999, 0.7], rot_dims=32, mlp=moe(8, 2, 128, shared=256)),
        ret(2, 128, 64, [0.96, 1.0], rot_dims=128, mlp=dense(384)),
    ], emb=4.0, logit_scale=0.5, cap=20.0),
}


def make_weights(cfg, seed, spread=1.0, decisive=False):
    """Matrices N(0, spread^2 / inputs) (queries and keys ``spread`` times wider, so that attention is peaked for
    spread > 1); norm weights and layer scales around 1; routers wide enough that the scores differ.

    ``decisive``: no choice of experts is a close call, so that rounding cannot flip one (a flipped choice moves a
    row, and every later row, by far more than rounding; bfloat16 runs are compared under such weights, float32 runs
    under the random routers). The last E entries of the stream (E: the most experts of a layer) hold a code of the
    token id, distinct levels in an order that turns with the id; no sublayer writes to them; expert e's router row
    reads entry e with a large factor beside small random entries."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    w = {}

    def mat(name, rows, cols, s=1.0):
        w[name] = torch.randn((rows, cols), generator=g) * (s / math.sqrt(cols))

    def around(name, n, centre=1.0, dev=0.2):
        w[name] = centre + dev * torch.randn((n,), generator=g)

    w["embed"] = torch.randn((V, W), generator=g) / cfg["embedding"]["scale"]
    for i, lay in enumerate(cfg["layers"]):
        p, m, q = "l%d" % i, lay["mixer"], "l%d.mix" % i
        around(p + ".norm1", W)
        around(p + ".ls1", W, 0.7, 0.2)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        if lay["type"] == "latent_attention":
            R, Q, dr = m["kv_rank"], m["q_rank"], m["rot_dim"]
            mat(q + ".dq", Q, W), around(q + ".dq.norm", Q), mat(q + ".uq", H * (d + dr), Q, spread * 1.5)
            if m.get("kv_from") is None:
                mat(q + ".dkv", R + dr, W, spread * 1.5), around(q + ".dkv.norm", R)
            mat(q + ".uk", H * d, R, spread), mat(q + ".uv", H * dv, R)
        else:
            mat(q + ".q", H * d, W, spread), mat(q + ".k", H * d, W, spread), mat(q + ".v", H * dv, W)
        mat(q + ".g", H * dv, W), mat(q + ".o", W, H * dv)
        mlp = lay["mlp"]
        if mlp is None:
            continue
        around(p + ".ls2", W, 0.7, 0.2)
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            mat(p + ".mlp.gate", F, W), mat(p + ".mlp.up", F, W), mat(p + ".mlp.down", W, F)
        else:
            F = mlp["expert"]["ff"]
            mat(p + ".mlp.router", mlp["router"]["experts"], W, 2.0)
            for e in range(mlp["router"]["experts"]):
                x = "%s.mlp.e%d" % (p, e)
                mat(x + ".gate", F, W, 1.5), mat(x + ".up", F, W, 1.5), mat(x + ".down", W, F)
            if mlp.get("shared"):
                F = mlp["shared"]["ff"]
                x = p + ".mlp.shared"
                mat(x + ".gate", F, W), mat(x + ".up", F, W), mat(x + ".down", W, F), mat(x + ".sg", 1, W, 2.0)
    around("final.norm", W)
    most = max([lay["mlp"]["router"]["experts"] for lay in cfg["layers"]
                if lay["mlp"] is not None and lay["mlp"]["kind"] == "moe"], default=0)
    if decisive and most:
        code = list(range(W - most, W))
        # (levels between -1.5 and 1.5 in the stream, so that the code does not outweigh the rest of a row)
        levels = torch.linspace(-1.5, 1.5, most) / cfg["embedding"]["scale"] if most > 1 else torch.zeros(1)
        for t in range(V):
            w["embed"][t, code] = torch.roll(levels, t % most)
        for name in list(w):
            if name.endswith(".o") or name.endswith(".down"):
                w[name][code, :] = 0.0
            elif name.endswith(".router"):
                w[name] *= 0.1
                for e in range(w[name].shape[0]):
                    w[name][e, code[e]] += 10.0
            elif name.endswith(".norm1"):
                w[name][code] = 1.0
    # the values a bfloat16 checkpoint holds, so that every run sees the same numbers
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}


def write_model(folder, cfg, weights):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def make_model(tmp_path, which, seed=0, spread=1.0, weights=None, decisive=False):
    cfg = CONFIGS[which] if isinstance(which, str) else which
    weights = weights if weights is not None else make_weights(cfg, seed, spread, decisive)
    tag = which if isinstance(which, str) else "custom"
    folder = write_model(os.path.join(str(tmp_path), "zevetar_%s_%d_%g_%d" % (tag, seed, spread, decisive)), cfg, weights)
    return folder, cfg, weights


def plain_logits(cfg, weights, tokens, dtype=torch.float64, storage=None):
    return P.forward(cfg, weights, tokens, dtype=dtype, storage=storage).to(torch.float32)


def bfloat16_limits(cfg, weights, tokens, ref, draws=3):
    """What rounding to bfloat16 may cost at every position: three times what it costs the plain implementation when
    it rounds what an engine may keep in 16 bits, the largest of ``draws`` draws of the rounding errors (the first
    rounds to nearest, the others move every value by up to half a step first: where a head's norm divides by a sum that
    nearly cancels, one draw says little), but no less than three times the median of the first draw over the
    positions."""
    e = row_errs(plain_logits(cfg, weights, tokens, dtype=torch.float32, storage=torch.bfloat16), ref)
    worst = torch.maximum(e, e.median())
    for i in range(1, draws):
        gen = torch.Generator().manual_seed(1000 + i)
        worst = torch.maximum(worst, row_errs(plain_logits(cfg, weights, tokens, dtype=torch.float32,
                                                           storage=(torch.bfloat16, gen)), ref))
    return 3.0 * worst


def single_layer(which, index, vocab=47):
    """The configuration of one layer of ``which`` alone (a mechanism on its own; a reader becomes an owner)."""
    cfg = CONFIGS[which]
    lay = json.loads(json.dumps(cfg["layers"][index]))
    lay["mixer"].pop("kv_from", None)
    out = dict(cfg)
    out.update(vocab=vocab, layers=[lay])
    return out
