"""Plain torch stand-ins for the HIP kernels, one per kernel, with the kernels' interface.

Two uses, both in tests only (the package itself has no such path and refuses to run without
its HIP library):
- the reference each kernel is compared with on the GPU;
- a way to run the host side of the engine (cache manager, step function, scheduler, replay)
  on a machine without GPU, by handing this object to the Runtime in place of the kernels.

Everything computes in float32 and rounds to the storage dtype at the end, like the kernels.
"""
import math

import numpy as np
import torch


# ---------------------------------------------------------------- counter-based noise (same as sampling.hip)

def _philox_first(c0, c1, k0, k1, c2=0, c3=0):
    """First output word of Philox4x32-10 for counters (c0, c1, c2, c3) and key (k0, k1); numpy uint64 maths."""
    M0, M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    mask = np.uint64(0xFFFFFFFF)
    c0 = c0.astype(np.uint64)
    c1 = np.full_like(c0, c1, dtype=np.uint64)
    c2 = np.full_like(c0, c2, dtype=np.uint64)
    c3 = np.full_like(c0, c3, dtype=np.uint64)
    k0 = np.uint64(k0)
    k1 = np.uint64(k1)
    for _ in range(10):
        p0 = M0 * c0
        p1 = M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & mask
        hi1, lo1 = p1 >> np.uint64(32), p1 & mask
        c0, c1, c2, c3 = (hi1 ^ c1 ^ k0) & mask, lo1, (hi0 ^ c3 ^ k1) & mask, lo0
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return c0


def gumbel_noise(seed, draw, V):
    """float32 [V]: -log(-log(u_i)), u_i = ((r_i >> 9) + 0.5) / 2^23, strictly inside (0, 1)."""
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    r = _philox_first(np.arange(V, dtype=np.uint64), int(draw) & 0xFFFFFFFF, seed & 0xFFFFFFFF, seed >> 32)
    u = ((r >> np.uint64(9)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)
    assert u.min() > 0.0 and u.max() < 1.0
    return torch.from_numpy(-np.log(-np.log(u))).to(torch.float32)


def _order_key(x):
    """Order-preserving uint32 image of float32 values (as int64 tensor)."""
    b = x.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    b = torch.where(b == 0x80000000, torch.zeros_like(b), b)      # -0 and +0 are one value
    neg = (b & 0x80000000) != 0
    return torch.where(neg, (~b) & 0xFFFFFFFF, b | 0x80000000)


class TorchOps:
    name = "torch-standin"

    # ------------------------------------------------------------ embedding / norm
    def embedding(self, ids, table, scale=1.0):
        return table[ids.long()].to(torch.float32) * scale

    def bad_token_seen(self):
        return False

    def patch_tokens(self, ids, src, prev):
        take = src[:ids.numel()] >= 0
        ids[take] = prev[src[:ids.numel()][take].long()].to(ids.dtype)

    def add_rms_norm(self, branch, residual, weight, eps, out_dtype, rows=None, weight_offset=0.0, defer_ok=False):
        x = None
        if branch is not None:
            x = branch.to(torch.float32)
        if residual is not None:
            x = residual if x is None else x + residual
        if branch is not None and residual is not None and rows is None:
            residual.copy_(x)
        if rows is not None:
            x = x[rows.long()]
        var = (x * x).mean(dim=-1, keepdim=True)
        y = x * torch.rsqrt(var + eps) * (weight.to(torch.float32) + weight_offset)
        return y.to(out_dtype)

    # ------------------------------------------------------------ rotary + cache write
    def rope_cache_write(self, qkv, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages):
        N = qkv.shape[0]
        q = qkv[:, :nh * d].reshape(N, nh, d)
        k = qkv[:, nh * d:(nh + nkv) * d].reshape(N, nkv, d)
        v = qkv[:, (nh + nkv) * d:(nh + 2 * nkv) * d].reshape(N, nkv, d)
        if table is not None:
            half = rot_dim // 2
            cs = table[positions.long()]
            cos, sin = cs[:, None, :half], cs[:, None, half:]

            def rot(x):
                x32 = x.to(torch.float32)
                out = x32.clone()
                if neox:
                    a, b = x32[..., :half], x32[..., half:rot_dim]
                    out[..., :half] = a * cos - b * sin
                    out[..., half:rot_dim] = b * cos + a * sin
                else:
                    a, b = x32[..., 0:rot_dim:2], x32[..., 1:rot_dim:2]
                    out[..., 0:rot_dim:2] = a * cos - b * sin
                    out[..., 1:rot_dim:2] = b * cos + a * sin
                return out.to(x.dtype)

            q, k = rot(q), rot(k)
            qkv[:, :nh * d] = q.reshape(N, nh * d)
            qkv[:, nh * d:(nh + nkv) * d] = k.reshape(N, nkv * d)
        if slots is not None:
            ps = k_pages.shape[2]
            sl = slots.long()
            ok = sl >= 0
            page, off = sl[ok] // ps, sl[ok] % ps
            k_pages[page, :, off, :] = k[ok]
            v_pages[page, :, :, off] = v[ok]

    def qkv_rope_cache(self, x, weight, bias, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages):
        y = self.linear(x, weight, bias)
        if table is not None or slots is not None:
            self.rope_cache_write(y, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages)
        return y

    # ------------------------------------------------------------ attention
    def paged_attention(self, q, k_pages, v_pages, block_tables, seg, pos, nh, nkv, d, scale, window=0, batch=None,
                        kernel=None, chunk=0, weights_f32=False, softcap=0.0):
        N = q.shape[0]
        ps = k_pages.shape[2]
        out = torch.empty((N, nh * d), dtype=q.dtype, device=q.device)
        rep = nh // nkv
        for t in range(N):
            s, p = int(seg[t]), int(pos[t])
            lo = max(0, p - window + 1) if window and window > 0 else 0
            if chunk:
                lo = p - p % chunk
            js = torch.arange(lo, p + 1, device=q.device)
            pages = block_tables[s].long()[js // ps]
            keys = k_pages[pages, :, js % ps, :].to(torch.float32)      # [n, nkv, d]
            vals = v_pages[pages, :, :, js % ps].to(torch.float32)      # [n, nkv, d]
            qt = q[t, :nh * d].to(torch.float32).reshape(nh, d)
            keys = keys.repeat_interleave(rep, dim=1)                    # [n, nh, d]
            vals = vals.repeat_interleave(rep, dim=1)
            sc = torch.einsum("hd,nhd->hn", qt, keys) * scale
            if softcap and softcap > 0:
                sc = softcap * torch.tanh(sc / softcap)
            pr = torch.softmax(sc, dim=-1)
            out[t] = torch.einsum("hn,nhd->hd", pr, vals).reshape(nh * d).to(q.dtype)
        return out

    # ------------------------------------------------------------ norm in groups, latent attention, experts
    @staticmethod
    def _gn(v, w, groups, eps):
        n, W = v.shape
        p = v.reshape(n, groups, W // groups)
        return (p / torch.sqrt((p * p).mean(dim=-1, keepdim=True) + eps)).reshape(n, W) * w

    def group_norm(self, x=None, x_weight=None, residual=None, out_weight=None, groups=1, x_eps=1e-5, out_eps=1e-5,
                   out_dtype=None, rows=None, history=None, index=0, mix=None, want_out=True):
        ref = x if x is not None else residual
        r = None
        if x is not None:
            r = self._gn(x.to(torch.float32), x_weight, groups, x_eps)
        if residual is not None:
            base = residual if rows is None else residual[rows.long()]
            r = base if r is None else base + r
            if x is not None and rows is None and history is None:
                residual.copy_(r)
        if history is not None:
            history[index].copy_(r)
            r = sum(mix[j] * history[j] for j in range(index + 1))
            residual.copy_(r)
        if not want_out:
            return None
        if out_weight is not None:
            r = self._gn(r, out_weight, groups, out_eps)
        return r.to(out_dtype or ref.dtype)

    @staticmethod
    def _rotate(v, cs, rot):
        half = rot // 2
        c, s = cs[..., :half], cs[..., half:rot]
        a, b = v[..., :half], v[..., half:rot]
        return torch.cat([a * c - b * s, b * c + a * s, v[..., rot:]], dim=-1)

    def latent_cache_write(self, x, weight, eps, rank, rot_width, positions, table, slots, k_pages, v_pages,
                           also_norm=None, also_weight=None):
        ps, D = k_pages.shape[2], k_pages.shape[3]
        xf = x.to(torch.float32)
        c = self._gn(xf[:, :rank], weight, 1, eps)
        r = self._rotate(xf[:, rank:rank + rot_width], table[positions.long()], table.shape[1])
        row = torch.zeros((x.shape[0], D), dtype=torch.float32)
        row[:, :rank], row[:, rank:rank + rot_width] = c, r
        row = row.to(k_pages.dtype)
        for n in range(x.shape[0]):
            s = int(slots[n])
            if s >= 0:
                k_pages[s // ps, 0, s % ps, :] = row[n]
                v_pages[s // ps, 0, :, s % ps] = row[n]
        if also_norm is not None:
            return self._gn(also_norm.to(torch.float32), also_weight, 1, eps).to(x.dtype)
        return None

    def head_linear(self, x, x_head, weight, out, out_head, gate=None, rope_tail=None, gate_wide=False):
        H, O, K = weight.shape
        if rope_tail is not None:
            x_at, out_at, width, positions, table = rope_tail
            self.rope_tail(x, x_head, x_at, out, out_head, out_at, H, width, positions, table)
        for h in range(H):
            y = x[:, h * x_head:h * x_head + K].to(torch.float32) @ weight[h].to(torch.float32).t()
            if gate is not None:
                g = gate[:, h * O:(h + 1) * O] if gate_wide else gate[:, h:h + 1]
                y = y * torch.sigmoid(g.to(torch.float32))
            out[:, h * out_head:h * out_head + O] = y.to(out.dtype)
        return out

    def rope_tail(self, x, x_head, x_at, out, out_head, out_at, heads, width, positions, table):
        cs = table[positions.long()]
        for h in range(heads):
            v = x[:, h * x_head + x_at:h * x_head + x_at + width].to(torch.float32)
            out[:, h * out_head + out_at:h * out_head + out_at + width] = self._rotate(v, cs, table.shape[1]).to(out.dtype)
            out[:, h * out_head + out_at + width:(h + 1) * out_head] = 0

    def table_moe(self, h, w_gate_up, w_down, token_ids, table, weight, base=None, pair_scale=None, base_scale=None,
                  out_scale=None, gated=True):
        F = w_gate_up.shape[1] // 2 if gated else w_gate_up.shape[1]
        out = torch.zeros(h.shape, dtype=torch.float32)
        for n in range(h.shape[0]):
            for k, e in enumerate(table[int(token_ids[n]) if token_ids is not None else n].tolist()):
                x = h[n].to(torch.float32) * (float(pair_scale[n, k]) if pair_scale is not None else 1.0)
                gu = (w_gate_up[e].to(torch.float32) @ x).to(h.dtype).to(torch.float32)
                if gated:
                    a = (gu[:F] / (1.0 + torch.exp(-gu[:F])) * gu[F:]).to(h.dtype).to(torch.float32)
                else:
                    a = (torch.relu(gu) ** 2).to(h.dtype).to(torch.float32)
                out[n] += (w_down[e].to(torch.float32) @ a) * (float(out_scale[n, k]) if out_scale is not None else 1.0)
        out = out * weight
        if base is not None:
            b = base.to(torch.float32)
            out = out + (b * base_scale[:, None] if base_scale is not None else b)
        return out.to(h.dtype)

    def moe_route(self, logits, experts, top, renorm=False, extra=-1):
        s = torch.sigmoid(logits[:, :experts])
        # the largest first, the lower index among equals
        order = torch.argsort(-logits[:, :experts], dim=-1, stable=True)[:, :top]
        w = torch.gather(s, 1, order)
        if renorm:
            w = w / w.sum(-1, keepdim=True)
        gate = torch.sigmoid(logits[:, extra]).contiguous() if extra >= 0 else None
        return order.to(torch.int32).contiguous(), w.contiguous(), gate

    # ------------------------------------------------------------ a token's extras, norms and rotated values, delta rule
    def moe_route_groups(self, logits, experts, top, softmax=True, groups=1, keep=1, renorm=False):
        z = logits[:, :experts].to(torch.float32)
        sc = torch.softmax(z, -1) if softmax else torch.sigmoid(z)
        N = z.shape[0]
        per = experts // groups
        best = z.reshape(N, groups, per).max(-1).values
        kept = torch.zeros((N, groups), dtype=torch.bool)
        kept.scatter_(1, torch.topk(best, keep, -1).indices, True)
        masked = z.masked_fill(~kept.repeat_interleave(per, 1), float("-inf"))
        choice = torch.topk(masked, top, -1).indices
        w = torch.gather(sc, 1, choice)
        if renorm:
            w = w / w.sum(-1, keepdim=True)
        return choice.to(torch.int32), w.contiguous()

    def hashed_pair_embedding(self, batch, table, pairs, prev_state, mul_prev, mul_cur, keep=False):
        ids = batch.token_ids.long()
        buckets = pairs.shape[0] - 1
        rows = torch.empty_like(ids)
        for t0, t1, slot in self._segments(batch):
            for t in range(t0, t1):
                if int(batch.positions[t]) == 0:
                    rows[t] = buckets
                    continue
                prev = int(prev_state[slot]) if t == t0 else int(ids[t - 1])
                rows[t] = (prev * int(mul_prev) + int(ids[t]) * int(mul_cur)) % buckets
            if t1 > t0:
                prev_state[slot] = int(ids[t1 - 1])
        out = table[ids].to(torch.float32) + pairs[rows].to(torch.float32)
        return (out, out.clone()) if keep else out

    def concat_rows(self, a, b, out_dtype):
        return torch.cat([a, b], -1).to(out_dtype)

    def gate_table(self, z, ids, table, at):
        zf = z.to(torch.float32)
        g = 0.5 * zf * (1.0 + torch.tanh(0.7978845608028654 * (zf + 0.044715 * zf ** 3)))
        return (g * table[ids.long()][:, at:at + z.shape[1]].to(torch.float32)).to(z.dtype)

    def relu_squared(self, z):
        return (torch.relu(z.to(torch.float32)) ** 2).to(z.dtype)

    @staticmethod
    def _turn(x, cs, interleaved, sign=1.0):
        """x [..., n] turned in pairs by the angles of cs [..., n] = [cos | sin] (broadcast over heads)."""
        n = cs.shape[-1]
        c, s = cs[..., :n // 2], cs[..., n // 2:] * sign
        out = x.clone()
        if interleaved:
            a, b = x[..., 0:n:2], x[..., 1:n:2]
            out[..., 0:n:2] = a * c - b * s
            out[..., 1:n:2] = b * c + a * s
        else:
            a, b = x[..., :n // 2], x[..., n // 2:n]
            out[..., :n // 2] = a * c - b * s
            out[..., n // 2:n] = b * c + a * s
        return out

    def attn_prepare_normed(self, q, k, v, heads, kv_heads, dim, vdim, padded, positions, slots, k_pages, v_pages,
                            q_weight=None, k_weight=None, eps=1e-5, table=None, table_v=None, interleaved=False,
                            v_norm=False):
        N = q.shape[0]
        qf = q[:, :heads * dim].to(torch.float32)
        kf = k[:, :kv_heads * dim].to(torch.float32)
        vf = v[:, :kv_heads * vdim].to(torch.float32).reshape(N, kv_heads, vdim)
        if q_weight is not None:
            qf = qf / torch.sqrt((qf * qf).mean(-1, keepdim=True) + eps) * q_weight
        if k_weight is not None:
            kf = kf / torch.sqrt((kf * kf).mean(-1, keepdim=True) + eps) * k_weight
        qf, kf = qf.reshape(N, heads, dim), kf.reshape(N, kv_heads, dim)
        if table is not None:
            rot = table.shape[1]
            cs = table[positions.long()][:, None, :]
            qf = torch.cat([self._turn(qf[..., :rot], cs, interleaved), qf[..., rot:]], -1)
            kf = torch.cat([self._turn(kf[..., :rot], cs, interleaved), kf[..., rot:]], -1)
        if v_norm:
            vf = vf / torch.sqrt((vf * vf).mean(-1, keepdim=True) + eps)
        if table_v is not None:
            vf = self._turn(vf, table_v[positions.long()][:, None, :], interleaved)
        out = torch.zeros((N, heads, padded), dtype=q.dtype)
        out[..., :dim] = qf.to(q.dtype)
        if slots is not None:
            ps = k_pages.shape[2]
            sl = slots.long()
            ok = sl >= 0
            page, off = sl[ok] // ps, sl[ok] % ps
            kp = torch.zeros((N, kv_heads, padded), dtype=q.dtype)
            kp[..., :dim] = kf.to(q.dtype)
            vp = torch.zeros((N, kv_heads, padded), dtype=q.dtype)
            vp[..., :vdim] = vf.to(q.dtype)
            k_pages[page, :, off, :] = kp[ok]
            v_pages[page, :, :, off] = vp[ok]
        return out.reshape(N, heads * padded)

    def attn_finish(self, a, padded, heads, vdim, positions, gate=None, table_v=None, interleaved=False):
        N = a.shape[0]
        x = a[:, :heads * padded].to(torch.float32).reshape(N, heads, padded)[..., :vdim]
        if table_v is not None:
            x = self._turn(x, table_v[positions.long()][:, None, :], interleaved, sign=-1.0)
        if gate is not None:
            x = x * torch.sigmoid(gate[:, :heads].to(torch.float32))[:, :, None]
        return x.reshape(N, heads * vdim).to(a.dtype)

    def gated_delta_state_floats(self, heads, dim, vdim):
        return heads * dim * vdim

    def gated_delta(self, qkv, q_at, k_at, v_at, a, dt_bias, a_log, b, state, batch, heads, kv_heads, dim, vdim,
                    q_scale, unit_eps=1e-6):
        N = qkv.shape[0]
        rep = heads // kv_heads
        q = qkv[:, q_at:q_at + kv_heads * dim].to(torch.float32).reshape(N, kv_heads, dim)
        k = qkv[:, k_at:k_at + kv_heads * dim].to(torch.float32).reshape(N, kv_heads, dim)
        v = qkv[:, v_at:v_at + heads * vdim].to(torch.float32).reshape(N, heads, vdim)
        q = (q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps) * q_scale).repeat_interleave(rep, 1)
        k = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)).repeat_interleave(rep, 1)
        beta = torch.sigmoid(b[:, :heads])
        g = torch.exp(-torch.exp(a_log)[None, :, None] * torch.nn.functional.softplus(
            a[:, :heads * dim] + dt_bias).reshape(N, heads, dim))
        out = torch.zeros((N, heads, vdim), dtype=torch.float32)
        for t0, t1, slot in self._segments(batch):
            S = state[slot, :heads * dim * vdim].reshape(heads, dim, vdim).clone()
            for t in range(t0, t1):
                S = S * g[t][:, :, None]
                u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
                S = S + k[t][:, :, None] * u[:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", S, q[t])
            state[slot, :heads * dim * vdim] = S.reshape(-1)
        return out.reshape(N, heads * vdim)

    def head_rms_gate(self, raw, heads, vdim, eps, weight, gate, out_dtype, activation="sigmoid"):
        N = raw.shape[0]
        x = raw[:, :heads * vdim].reshape(N, heads, vdim)
        y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        if weight is not None:
            y = y * weight
        if gate is not None:
            g = gate[:, :heads * vdim].to(torch.float32).reshape(N, heads, vdim)
            y = y * (torch.sigmoid(g) if activation == "sigmoid" else g * torch.sigmoid(g))
        return y.reshape(N, heads * vdim).to(out_dtype)

    def scale_add_norm(self, a, scale_a, b, scale_b, residual, weight=None, eps=1e-5):
        r = residual + scale_a * a.to(torch.float32)
        if b is not None:
            r = r + scale_b * b.to(torch.float32)
        residual.copy_(r)
        if weight is None:
            return None
        return (r / torch.sqrt((r * r).mean(-1, keepdim=True) + eps) * weight.to(torch.float32)).to(a.dtype)

    def logit_cap(self, logits, scale=1.0, cap=0.0):
        y = logits * scale
        logits.copy_(cap * torch.tanh(y / cap) if cap > 0 else y)
        return logits

    def retention_state_floats(self, heads, dim, vdim):
        return heads * dim * vdim

    def retention(self, q, k, v, decay, out_gate, state, batch, heads, dim, vdim, k_scale, eps, table=None):
        H, d, dv = heads, dim, vdim
        out = torch.empty((q.shape[0], H * dv), dtype=q.dtype)
        g = decay[:H]
        for a, b, slot in self._segments(batch):
            S = state[slot, :H * d * dv].reshape(H, d, dv).clone()
            for t in range(a, b):
                qt = q[t, :H * d].to(torch.float32).reshape(H, d)
                kt = k[t, :H * d].to(torch.float32).reshape(H, d)
                if table is not None:
                    cs = table[int(batch.positions[t])]
                    qt, kt = self._rotate(qt, cs, table.shape[1]), self._rotate(kt, cs, table.shape[1])
                vt = v[t, :H * dv].to(torch.float32).reshape(H, dv)
                S = g[:, None, None] * S + (kt * k_scale)[:, :, None] * vt[:, None, :]
                o = torch.einsum("hdv,hd->hv", S, qt)
                o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
                gt = out_gate[t, :H * dv].to(torch.float32)
                out[t] = (o.reshape(-1) * (gt / (1.0 + torch.exp(-gt)))).to(q.dtype)
            state[slot, :H * d * dv] = S.reshape(-1)
        return out

    # ------------------------------------------------------------ Dynamic Tanh, state-carrying mixers
    def dyt_norm(self, branch, residual, weight, bias, alpha, out_dtype, rows=None):
        x = None
        if branch is not None:
            x = branch.to(torch.float32)
        if residual is not None:
            x = residual if x is None else x + residual
        if branch is not None and residual is not None and rows is None:
            residual.copy_(x)
        if rows is not None:
            x = x[rows.long()]
        return (torch.tanh(alpha * x) * weight + bias).to(out_dtype)

    @staticmethod
    def _segments(batch):
        starts = [int(v) for v in batch.seg_starts[:batch.n_segments + 1]]
        slots = [int(v) for v in batch.state_slots[:batch.n_segments]]
        return [(starts[i], starts[i + 1], slots[i]) for i in range(batch.n_segments)]

    def short_conv(self, u, weight, bias, state, batch, activation=None):
        C, taps = weight.shape
        w = weight.to(torch.float32)
        out = torch.empty((u.shape[0], C), dtype=u.dtype)
        for a, b, slot in self._segments(batch):
            old = state[slot, :C * (taps - 1)].reshape(C, taps - 1).t() if taps > 1 else torch.zeros(0, C)
            seq = torch.cat([old, u[a:b].to(torch.float32)], 0)             # [taps - 1 + n, C]
            y = sum(seq[j:j + (b - a)] * w[:, j] for j in range(taps))
            if bias is not None:
                y = y + bias.to(torch.float32)
            if activation == "silu":
                y = y / (1.0 + torch.exp(-y))
            out[a:b] = y.to(u.dtype)
            if taps > 1:
                state[slot, :C * (taps - 1)] = seq[seq.shape[0] - (taps - 1):].t().reshape(-1)
        return out

    def selective_scan(self, x, dt, bc, b_at, c_at, z, a_log, d_skip, state, batch):
        inner, n = a_log.shape
        A = -torch.exp(a_log)
        y = torch.empty((x.shape[0], inner), dtype=x.dtype)
        for a, b, slot in self._segments(batch):
            S = state[slot, :inner * n].reshape(inner, n).clone()
            for t in range(a, b):
                d = torch.nn.functional.softplus(dt[t], threshold=20.0)
                xt, zt = x[t].to(torch.float32), z[t, :inner].to(torch.float32)
                B, Cc = bc[t, b_at:b_at + n].to(torch.float32), bc[t, c_at:c_at + n].to(torch.float32)
                S = torch.exp(d[:, None] * A) * S + (d * xt)[:, None] * B[None, :]
                y[t] = ((S @ Cc + d_skip * xt) * (zt / (1.0 + torch.exp(-zt)))).to(x.dtype)
            state[slot, :inner * n] = S.reshape(-1)
        return y

    def mlstm_state_floats(self, heads, dim, vdim):
        return heads * dim * (vdim + 1) + heads

    def mlstm(self, q, k, v, gates, out_gate, norm_weight, state, batch, heads, dim, vdim, q_scale, gate_cap, eps):
        H, d, dv = heads, dim, vdim
        out = torch.empty((q.shape[0], H * dv), dtype=q.dtype)
        nS = H * d * (dv + 1)
        for a, b, slot in self._segments(batch):
            Sx = state[slot, :nS].reshape(H, d, dv + 1).clone()              # S, and n as the last column
            m = state[slot, nS:nS + H].clone()
            for t in range(a, b):
                qt = q[t, :H * d].to(torch.float32).reshape(H, d) * q_scale
                kt = k[t, :H * d].to(torch.float32).reshape(H, d)
                vt = torch.cat([v[t, :H * dv].to(torch.float32).reshape(H, dv), torch.ones(H, 1)], 1)
                gi = gate_cap * torch.tanh(gates[t, :H] / gate_cap)
                gf = torch.nn.functional.logsigmoid(gate_cap * torch.tanh(gates[t, H:2 * H] / gate_cap))
                m_new = torch.maximum(gf + m, gi)
                keep, take = torch.exp(gf + m - m_new), torch.exp(gi - m_new)
                m = m_new
                Sx = keep[:, None, None] * Sx + take[:, None, None] * kt[:, :, None] * vt[:, None, :]
                ox = torch.einsum("hdv,hd->hv", Sx, qt)
                o = ox[:, :dv] / (torch.maximum(ox[:, dv].abs(), torch.exp(-m)) + 1e-6)[:, None]
                o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
                g = out_gate[t, :H * dv].to(torch.float32)
                out[t] = (o.reshape(-1) * norm_weight * torch.sigmoid(g)).to(q.dtype)
            state[slot, :nS] = Sx.reshape(-1)
            state[slot, nS:nS + H] = m
        return out

    def attn_prepare(self, q, k, v, heads, kv_heads, dim, vdim, padded, positions, slots, k_pages, v_pages, table=None,
                     unit_norm_eps=None, temp_coef=0.0, temp_every=0):
        N = q.shape[0]
        qf = q[:, :heads * dim].to(torch.float32).reshape(N, heads, dim)
        kf = k[:, :kv_heads * dim].to(torch.float32).reshape(N, kv_heads, dim)
        if unit_norm_eps is not None:
            qf = qf / torch.sqrt((qf * qf).mean(-1, keepdim=True) + unit_norm_eps)
            kf = kf / torch.sqrt((kf * kf).mean(-1, keepdim=True) + unit_norm_eps)
        if table is not None:
            rot = table.shape[1]
            cs = table[positions.long()][:, None, :]
            qf = torch.cat([self._rotate(qf[..., :rot], cs, rot), qf[..., rot:]], -1)
            kf = torch.cat([self._rotate(kf[..., :rot], cs, rot), kf[..., rot:]], -1)
        if temp_every:
            p = positions.to(torch.float32)
            qf = qf * (1.0 + temp_coef * torch.log(torch.floor((p + 1) / temp_every) + 1.0))[:, None, None]
        out = torch.zeros((N, heads, padded), dtype=q.dtype)
        out[..., :dim] = qf.to(q.dtype)
        if slots is not None:
            ps = k_pages.shape[2]
            sl = slots.long()
            ok = sl >= 0
            page, off = sl[ok] // ps, sl[ok] % ps
            kp = torch.zeros((N, kv_heads, padded), dtype=q.dtype)
            kp[..., :dim] = kf.to(q.dtype)
            vp = torch.zeros((N, kv_heads, padded), dtype=q.dtype)
            vp[..., :vdim] = v[:, :kv_heads * vdim].reshape(N, kv_heads, vdim)
            k_pages[page, :, off, :] = kp[ok]
            v_pages[page, :, :, off] = vp[ok]
        return out.reshape(N, heads * padded)

    def head_gate(self, x, x_head, heads, vdim, gate=None):
        N = x.shape[0]
        y = x[:, :heads * x_head].reshape(N, heads, x_head)[..., :vdim].reshape(N, heads * vdim).to(torch.float32)
        if gate is not None:
            y = y * torch.sigmoid(gate[:, :heads * vdim].to(torch.float32))
        return y.to(x.dtype)

    def rms_pair(self, a, b, wa, wb, eps, scale=0.5):
        a32, b32 = a.to(torch.float32), b.to(torch.float32)
        na = a32 / torch.sqrt((a32 * a32).mean(-1, keepdim=True) + eps) * wa
        nb = b32 / torch.sqrt((b32 * b32).mean(-1, keepdim=True) + eps) * wb
        return (scale * (na + nb)).to(a.dtype)

    # ------------------------------------------------------------ feed-forward / linear
    def gated_act(self, gu, kind="silu"):
        I = gu.shape[1] // 2
        g, u = gu[:, :I].to(torch.float32), gu[:, I:].to(torch.float32)
        if kind == "silu":
            a = g / (1.0 + torch.exp(-g))
        elif kind == "gelu":
            a = 0.5 * g * (1.0 + torch.erf(g / math.sqrt(2.0)))
        elif kind == "gelu_tanh":
            a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
        else:
            raise ValueError(kind)
        return (a * u).to(gu.dtype)

    def linear_gated(self, x, weight, bias=None, kind="silu"):
        return self.gated_act(self.linear(x, weight, bias), kind)

    def linear(self, x, weight, bias=None, out_dtype=None, pending_ok=False, out=None):
        y = x.to(torch.float32) @ weight.to(torch.float32).t()
        if bias is not None:
            y = y + bias.to(torch.float32)
        y = y.to(out_dtype or x.dtype)
        return y if out is None else out.copy_(y)

    def linear_wide(self, x, weight, bias=None, out=None):
        y = self.linear(x, weight, bias, out_dtype=torch.float32)
        return y if out is None else out.copy_(y)

    def materialize(self, y):
        return y

    # ------------------------------------------------------------ sampling
    def sample(self, logits, temperature=None, top_k=None, top_p=None, min_p=None, seeds=None, draws=None):
        R, V = logits.shape
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        for r in range(R):
            T = float(temperature[r]) if temperature is not None else 0.0
            row = logits[r].to(torch.float32).cpu()
            if T < 1e-5:
                out[r] = int(torch.argmax(row))      # first maximum
                continue
            x = row * np.float32(1.0 / np.float32(T))
            keys = _order_key(x)
            mx = x.max()
            cut = 0
            k = int(top_k[r]) if top_k is not None else -1
            if 0 < k < V:
                cut = int(torch.sort(keys, descending=True).values[k - 1])
            p = float(top_p[r]) if top_p is not None else 1.0
            if p < 1.0:
                e = torch.where(keys >= cut, torch.exp(x - mx), torch.zeros_like(x))
                target = np.float32(p) * e.sum()
                order = torch.argsort(keys, descending=True)
                csum = torch.cumsum(e[order], dim=0)
                # largest key whose mass of keys >= it reaches the target (ties counted together)
                sk = keys[order]
                group_end = torch.cat([sk[1:] != sk[:-1], torch.ones(1, dtype=torch.bool)])
                hit = torch.nonzero(group_end & (csum >= target))
                best = max(cut, int(sk[int(hit[0])])) if hit.numel() else cut
                cut = best
            mp = float(min_p[r]) if min_p is not None else 0.0
            if mp > 0.0:
                c = int(_order_key((mx + np.float32(math.log(mp))).reshape(1))[0])
                cut = max(cut, c)
            cut = min(cut, int(_order_key(mx.reshape(1))[0]))
            seed = int(seeds[r]) if seeds is not None else 0
            draw = int(draws[r]) if draws is not None else 0
            y = x + gumbel_noise(seed, draw, V)
            y = torch.where(keys >= cut, y, torch.full_like(y, float("-inf")))
            out[r] = int(torch.argmax(y))
        return out

    def apply_penalties(self, logits, tokens, offsets, prompt_lens, presence, frequency, repetition):
        R, V = logits.shape
        for r in range(R):
            b, e, np_ = int(offsets[r]), int(offsets[r + 1]), int(prompt_lens[r])
            toks = tokens[b:e].long()
            seen = torch.zeros(V, dtype=torch.bool, device=logits.device)
            seen[toks] = True
            counts = torch.zeros(V, dtype=torch.float32, device=logits.device)
            counts.index_add_(0, toks[np_:], torch.ones(e - b - np_, device=logits.device))
            x = logits[r]
            rep = torch.where(seen, repetition[r], torch.ones_like(x))
            x = torch.where(x > 0, x / rep, x * rep)
            x = x - frequency[r] * counts
            x = x - presence[r] * (counts > 0).to(torch.float32)
            logits[r] = x
