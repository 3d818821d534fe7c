"""A plain, slow implementation of the Murulorn design: whole sequences, no cache, recurrences token by token, one
function per mechanism. It shares nothing with the package: it reads a configuration dictionary and a dictionary of
tensors by checkpoint name. ``dtype`` float64 gives the yardstick, float32 what float32 rounding costs; ``storage``
(a torch dtype, None, or a pair (dtype, generator) for another draw of the rounding errors) rounds what an engine may
keep in 16 bits: the operands and results of the projections, the convolutions and the activations between them.

Notation: T tokens, width W. A layer is x += n1b(mixer(n1(x))); x += n2b(ffn(n2(x))); x += side(x, token), every n an
RMS norm whose stored weight w acts as 1 + w. Layers ``start`` to ``stop`` - 1 of the list run ``times`` times with the
same weights; each such pass begins with x = M [x ; x0], x0 the embedding's output.
"""
import math

import torch


def _rt(x, storage):
    """Round to the storage type and back. ``storage`` may be (type, generator): the value is first moved by up to
    half a bfloat16 step at random, which gives another draw of the rounding errors."""
    if storage is None:
        return x
    if isinstance(storage, tuple):
        storage, gen = storage
        x = x * (1.0 + (torch.rand(x.shape, generator=gen, dtype=torch.float32).to(x.dtype) - 0.5) * 2.0 ** -8)
    return x.to(storage).to(x.dtype)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_squared(z):
    return torch.relu(z) ** 2


def linear(x, w, storage):
    return _rt(_rt(x, storage) @ w.T, storage)


# ---------------------------------------------------------------- embedding


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token: a hash of (previous, current); the first token takes the last row."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets)
    return rows


def embed(cfg, tw, tokens, dtype):
    b = cfg["embedding"]["bigram"]
    ids = torch.tensor(tokens, dtype=torch.long)
    rows = torch.tensor(bigram_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"]), dtype=torch.long)
    return tw["embed"].to(dtype)[ids] + tw["bigram"].to(dtype)[rows]


# ---------------------------------------------------------------- rotation


def turn_pairs(x, positions, dims, base, interleaved, sign=1.0):
    """x [T, heads, d]: the first ``dims`` entries of every head turned by sign * position * base^(-2i/dims) in pair
    i; pairs (2i, 2i + 1) if ``interleaved`` else (i, i + dims/2). The rest passes."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = (torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)).to(x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :] * sign
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
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


# ---------------------------------------------------------------- attention


def attention(m, tw, p, h, eps, storage, interleaved=True):
    """Softmax attention within a window, with: one RMS norm over all of q and one over all of k (weights of that
    size), partial rotation of q and k, values divided by their root mean square per head and turned by their own
    position over their whole width, scores bounded by cap tanh(s / cap), the summed values turned back by the
    query's position, one sigmoid gate a head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rms(linear(h, tw[p + ".q"].to(h.dtype), storage), eps) * tw[p + ".q.norm"].to(h.dtype)
    k = rms(linear(h, tw[p + ".k"].to(h.dtype), storage), eps) * tw[p + ".k.norm"].to(h.dtype)
    v = linear(h, tw[p + ".v"].to(h.dtype), storage).view(T, G, dv)
    rot = m["rot"]
    q = _rt(turn_pairs(q.view(T, H, d), pos, rot["dims"], rot["base"], interleaved), storage)
    k = _rt(turn_pairs(k.view(T, G, d), pos, rot["dims"], rot["base"], interleaved), storage)
    v = _rt(turn_pairs(rms(v, eps), pos, dv, rot["base"], interleaved), storage)
    gate = torch.sigmoid(linear(h, tw[p + ".g"].to(h.dtype), storage))            # [T, H]
    cap, size = m.get("softcap"), m["mask"]["size"]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    diff = pos[:, None] - pos[None, :]
    seen = (diff >= 0) & (diff < size)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~seen, float("-inf"))
        out[:, hd] = torch.softmax(s, -1) @ v[:, g]
    out = turn_pairs(_rt(out, storage), pos, dv, rot["base"], interleaved, sign=-1.0)
    out = _rt(out * gate[:, :, None], storage)
    return linear(out.reshape(T, H * dv), tw[p + ".o"].to(h.dtype), storage)


# ---------------------------------------------------------------- delta rule


def short_conv_silu(u, w, storage):
    """Causal filter per channel, zeros before the start, then SiLU. u [T, C], w [C, taps]; the last tap is the
    current token's."""
    T, C = u.shape
    taps = w.shape[1]
    u = _rt(u, storage)
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j][None, :]
    return _rt(y * torch.sigmoid(y), storage)


def delta_rule(q, k, v, beta, decay):
    """Per head, token by token: S <- diag(decay_t) S; u = beta_t (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t.
    q, k [T, H, d]; v [T, H, dv]; beta [T, H]; decay [T, H, d] (one factor a row of S). S starts at zero."""
    T, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=q.dtype)
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        S = S * decay[t][:, :, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def channel_delta(m, tw, p, h, eps, storage):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    dt = h.dtype

    def branch(name):
        return short_conv_silu(linear(h, tw[p + "." + name].to(dt), storage), tw[p + "." + name + ".conv"].to(dt), storage)

    q, k, v = branch("q").view(T, G, d), branch("k").view(T, G, d), branch("v").view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(linear(h, tw[p + ".b"].to(dt), storage))
    low = linear(linear(h, tw[p + ".a1"].to(dt), storage), tw[p + ".a2"].to(dt), storage)
    step = torch.nn.functional.softplus(low + tw[p + ".dt_bias"].to(dt)).view(T, H, d)
    decay = torch.exp(-torch.exp(tw[p + ".A_log"].to(dt))[None, :, None] * step)
    o = delta_rule(q, k, v, beta, decay)
    gate = torch.sigmoid(linear(linear(h, tw[p + ".g1"].to(dt), storage), tw[p + ".g2"].to(dt), storage)).view(T, H, dv)
    o = _rt(rms(o, eps) * tw[p + ".norm"].to(dt)[None, None, :] * gate, storage)
    return linear(o.reshape(T, H * dv), tw[p + ".o"].to(dt), storage)


# ---------------------------------------------------------------- feed-forward


def dense_ffn(tw, p, h, storage):
    a = _rt(relu_squared(linear(h, tw[p + ".up"].to(h.dtype), storage)), storage)
    return linear(a, tw[p + ".down"].to(h.dtype), storage)


def choose_experts(scores, top, groups, keep):
    """scores [T, E] -> chosen experts [T, top]: the largest scores among the experts of the ``keep`` groups (of
    ``groups`` equal groups of neighbours) whose best score is largest."""
    T, E = scores.shape
    per = E // groups
    best = scores.view(T, groups, per).max(-1).values
    kept = torch.topk(best, keep, -1).indices
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = scores.masked_fill(~allowed.repeat_interleave(per, 1), float("-inf"))
    return torch.topk(masked, top, -1).indices


def moe_ffn(mlp, tw, p, h, storage):
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    z = _rt(h, storage).to(torch.float32 if h.dtype != torch.float64 else h.dtype) @ tw[p + ".router"].to(
        torch.float32 if h.dtype != torch.float64 else h.dtype).T
    s = torch.softmax(z, -1)
    chosen = choose_experts(s, top, g["count"], g["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            y = dense_ffn(tw, "%s.e%d" % (p, e), h[t:t + 1], storage)[0]
            out[t] = out[t] + s[t, e].to(h.dtype) * y
    return _rt(out, storage)


# ---------------------------------------------------------------- the token's side input


def token_side(cfg, tw, layer, x, tokens, storage):
    dim = cfg["token_side"]["dim"]
    p = "l%d.side" % layer
    ids = torch.tensor(tokens, dtype=torch.long)
    e = tw["side.embed"].to(x.dtype)[ids][:, layer * dim:(layer + 1) * dim]
    g = _rt(gelu_tanh(linear(x, tw[p + ".gate"].to(x.dtype), storage)) * e, storage)
    y = linear(g, tw[p + ".proj"].to(x.dtype), storage)
    return x + rms(y, cfg["norm"]["eps"]) * tw[p + ".norm"].to(x.dtype)


# ---------------------------------------------------------------- the model


def layer_runs(cfg):
    """The order in which the layers run: (layer, first of a pass?)"""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, tw, tokens, dtype=torch.float64, storage=None, want_layers=False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer run)."""
    tw = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tw.items()}
    eps = cfg["norm"]["eps"]
    x0 = embed(cfg, tw, tokens, dtype)
    x = x0.clone()
    streams = []
    for li, first in layer_runs(cfg):
        layer = cfg["layers"][li]
        p = "l%d" % li
        if first:
            x = linear(torch.cat([x, x0], -1), tw["loop.in"], storage).to(dtype)
        h = _rt(norm_one_plus(x, tw[p + ".norm1"], eps), storage)
        if layer["type"] == "attention":
            a = attention(layer["mixer"], tw, p + ".mix", h, eps, storage)
        elif layer["type"] == "channel_delta":
            a = channel_delta(layer["mixer"], tw, p + ".mix", h, eps, storage)
        else:
            raise ValueError(layer["type"])
        x = x + norm_one_plus(a, tw[p + ".norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = _rt(norm_one_plus(x, tw[p + ".norm2"], eps), storage)
            f = dense_ffn(tw, p + ".mlp", h, storage) if mlp["kind"] == "dense" else moe_ffn(mlp, tw, p + ".mlp", h, storage)
            x = x + norm_one_plus(f, tw[p + ".norm2b"], eps)
        if cfg.get("token_side"):
            x = token_side(cfg, tw, li, x, tokens, storage)
        streams.append(x.clone())
    h = _rt(norm_one_plus(x, tw["final.norm"], eps), storage)
    logits = _rt(h, storage) @ _rt(tw["embed"], storage).T
    return (logits, torch.stack(streams)) if want_layers else logits
