"""A plain, slow implementation of the Zevetar design: whole sequences, no cache, recurrences token by token, one
function per mechanism. It shares nothing with the package: it reads a configuration dictionary and a dictionary of
tensors by checkpoint name. ``dtype`` float64 gives the yardstick, float32 what float32 rounding costs; ``storage``
(a torch dtype, None, or a pair (dtype, generator) for another draw of the rounding errors) rounds what an engine may
keep in 16 bits: the operands and results of the projections and the activations between them.

Notation: T tokens, width W. A layer is x += ls1 * mixer(h) + ls2 * ffn(h) with h = rms_norm(x; w1): one norm, both
sublayers read it, each result is scaled entry by entry before the sum.
"""
import math

import torch


def _rt(x, storage):
    """Round to the storage type and back (what a 16-bit buffer does to a value). ``storage`` may be (type, generator):
    the value is then moved by up to half a bfloat16 step at random before it is rounded, which gives another draw
    of the rounding errors (an engine that adds up in another order rounds some values the other way)."""
    if storage is None:
        return x
    if isinstance(storage, tuple):
        storage, gen = storage
        x = x * (1.0 + (torch.rand(x.shape, generator=gen, dtype=torch.float32).to(x.dtype) - 0.5) * 2.0 ** -8)
    return x.to(storage).to(x.dtype)


def rms_norm(x, w, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def linear(x, w, storage):
    """W x for every row of x, operands and result rounded as stored."""
    return _rt(_rt(x, storage) @ w.T, storage)


# ---------------------------------------------------------------- rotations


def rotary_frequencies(dims, base, scaling, dtype):
    """f_i = base^(-2i/dims), i < dims/2; with YaRN scaling the blend of f_i / factor and f_i along a ramp over i, and
    the factor by which cos and sin grow."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    grow = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def turn(t):
            return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

        lo = max(math.floor(turn(float(scaling["fast"]))), 0)
        hi = min(math.ceil(turn(float(scaling["slow"]))), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        grow = 0.1 * math.log(factor) + 1.0
    return f.to(dtype), grow


def rotate(x, positions, dims, base, scaling, interleaved):
    """x [T, heads, d]: the first ``dims`` entries of every head turned by the position; pairs (2i, 2i+1) if
    ``interleaved`` else (i, i + dims/2). The rest passes."""
    f, grow = rotary_frequencies(dims, base, scaling, x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]                      # [T, dims/2]
    c, s = (torch.cos(a) * grow)[:, None, :], (torch.sin(a) * grow)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    return out


# ---------------------------------------------------------------- mixers


def latent_kv(h, m, t, pre, eps, positions, storage):
    """What a layer with a latent of its own keeps per token: c [T, R] and the turned key part r [T, dr]."""
    R, dr = m["kv_rank"], m["rot_dim"]
    low = linear(h, t[pre + "dkv"], storage)
    c = _rt(rms_norm(low[:, :R], t[pre + "dkv.norm"], eps), storage)
    r = rotate(low[:, None, R:R + dr], positions, m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"), True)[:, 0]
    return c, _rt(r, storage)


def latent_attention(h, m, t, pre, eps, positions, kv, storage):
    """Softmax attention whose keys and values are up-projections of the latent ``kv`` = (c, r), within a window."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, r = kv
    cq = _rt(rms_norm(linear(h, t[pre + "dq"], storage), t[pre + "dq.norm"], eps), storage)
    q = linear(cq, t[pre + "uq"], storage).reshape(T, H, dn + dr)
    qn = q[..., :dn]
    qr = rotate(q[..., dn:], positions, m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"), True)
    kn = linear(c, t[pre + "uk"], storage).reshape(T, H, dn)
    v = linear(c, t[pre + "uv"], storage).reshape(T, H, dv)
    score = (torch.einsum("thd,uhd->htu", qn, kn) + torch.einsum("thd,ud->htu", qr, r)) * m["scale"]
    i, j = positions[:, None], positions[None, :]
    seen = (i - j >= 0)
    size = (m.get("mask") or {}).get("size")
    if size:
        seen = seen & (i - j < size)
    score = score.masked_fill(~seen[None], float("-inf"))
    p = torch.softmax(score, dim=-1)
    o = torch.einsum("htu,uhe->the", p, v).reshape(T, H * dv)
    o = _rt(_rt(o, storage) * torch.sigmoid(linear(h, t[pre + "g"], storage)), storage)
    return linear(o, t[pre + "o"], storage)


def retention(h, m, t, pre, eps, positions, storage, state=None):
    """Linear attention with a fixed decay per head: S <- decay S + k v^T, o = S^T q; every head's o over its root
    mean square, times silu(W_g h), then W_o. ``state`` [H, d, dv] (zeros at a sequence's start) is updated in place."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot")
    q = linear(h, t[pre + "q"], storage).reshape(T, H, d)
    k = linear(h, t[pre + "k"], storage).reshape(T, H, d)
    v = linear(h, t[pre + "v"], storage).reshape(T, H, dv)
    if rot:
        q = rotate(q, positions, rot["dims"], rot["base"], rot.get("scaling"), False)
        k = rotate(k, positions, rot["dims"], rot["base"], rot.get("scaling"), False)
    k = k * d ** -0.5
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, d, dv, dtype=h.dtype) if state is None else state
    o = torch.empty(T, H, dv, dtype=h.dtype)
    for n in range(T):
        S.mul_(decay[:, None, None]).add_(k[n][:, :, None] * v[n][:, None, :])
        o[n] = torch.einsum("hde,hd->he", S, q[n])
    o = rms_norm(o, None, eps).reshape(T, H * dv)
    o = _rt(o * silu(linear(h, t[pre + "g"], storage)), storage)
    return linear(o, t[pre + "o"], storage)


# ---------------------------------------------------------------- feed-forward


def gated_ffn(h, t, pre, storage):
    a = _rt(silu(linear(h, t[pre + "gate"], storage)) * linear(h, t[pre + "up"], storage), storage)
    return linear(a, t[pre + "down"], storage)


def routed_experts(h, mlp, t, pre, storage):
    """Scores sigmoid(W_r h) in the working precision; the ``top`` largest choose the experts; an expert gets its
    score times h as input; the shared expert's result times sigmoid(w_sg . h)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    hs = _rt(h, storage)
    z = hs @ t[pre + "router"].T
    # (the largest scores are the largest logits; chosen by the logits, two scores that both round to 1 stay apart)
    idx = torch.topk(z, top, dim=-1).indices
    w = torch.sigmoid(torch.gather(z, 1, idx))
    out = torch.zeros_like(h)
    for e in range(E):
        for kk in range(top):
            rows = (idx[:, kk] == e).nonzero()[:, 0]
            if len(rows):
                out[rows] += gated_ffn(w[rows, kk][:, None] * h[rows], t, "%se%d." % (pre, e), storage)
    if mlp.get("shared") is not None:
        g = torch.sigmoid(hs @ t[pre + "shared.sg"].T)                      # [T, 1]
        out = out + g * gated_ffn(h, t, pre + "shared.", storage)
    return _rt(out, storage)


# ---------------------------------------------------------------- the model


def forward(cfg, tensors, tokens, dtype=torch.float64, storage=None, layers_out=None):
    """Logits [T, vocab] of one whole sequence. ``layers_out``: a list that takes the stream after every layer."""
    t = {n: (x.to(dtype) if x.dtype.is_floating_point else x) for n, x in tensors.items()}
    eps = cfg["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    T = len(ids)
    positions = torch.arange(T)
    x = t["embed"][ids] * cfg["embedding"]["scale"]
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        pre = "l%d." % i
        m, mlp = layer["mixer"], layer.get("mlp")
        h = _rt(rms_norm(x, t[pre + "norm1"], eps), storage)
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_kv(h, m, t, pre + "mix.", eps, positions, storage)
                src = i
            a = latent_attention(h, m, t, pre + "mix.", eps, positions, latents[src], storage)
        elif layer["type"] == "retention":
            a = retention(h, m, t, pre + "mix.", eps, positions, storage)
        else:
            raise ValueError("layer type %r" % layer["type"])
        total = a * t[pre + "ls1"]
        if mlp is not None:
            f = gated_ffn(h, t, pre + "mlp.", storage) if mlp["kind"] == "dense" else \
                routed_experts(h, mlp, t, pre + "mlp.", storage)
            total = total + f * t[pre + "ls2"]
        x = x + total
        if layers_out is not None:
            layers_out.append(x.clone())
    h = _rt(rms_norm(x, t["final.norm"], eps), storage)
    logits = (h @ _rt(t["embed"], storage).T) * cfg["logit_scale"]
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(cfg, tensors, prompt, n, dtype=torch.float64):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, tensors, toks, dtype)[-1].argmax()))
    return toks[len(prompt):]
