"""Attention over a cached latent: keys and values of all heads are up-projections of one small vector per token.

Per token the layer keeps c = rms_norm(Wdkv h)[:R] (the latent) and r = rotate(Wdkv h)[R:R+dr] (one rotated key
part shared by the heads). Head h's key is [Uk_h c | r], its value Uv_h c, its query [qn_h | rotate(qr_h)] with
q = Wuq rms_norm(Wdq h). With the up-projections folded into the query and the output,

    score_h(t, j) = ((Uk_h^T qn_h(t)) . c(j) + qr_h(t) . r(j)) * scale,   out_h(t) = Uv_h sum_j p_h(t, j) c(j),

the attention runs on the cache as it is: one key/value head of width D = R + dr (rounded up to what the
attention kernels take) that all query heads share, through the paged attention kernels the other mixers use.
out_h is multiplied by sigmoid(Wg h)_h before the output projection (one gate a head, or with ``gate_per_entry`` one
for every entry of every head's value). A layer may read another layer's cache (the schedule's ``cache_from``): it
then has no down-projection to the latent, only its own up-projections. ``window``: a query sees itself and the
window - 1 positions before it; ``cache_window`` is what the pages are kept for (the widest window among the layers
that read them; None: everything). ``weights_f32``: the softmax weights stay float32 into the product with the cached
rows (``HipOps.paged_attention``), for a design that asks for it. A position encoding of style "gptj" (pairs
(2i, 2i + 1)) is served by the same kernels: the rows of Wuq and Wdkv that make the rotated entries are put in the order
(0, 2, 4, ..., 1, 3, 5, ...) at load, which changes no score (the same permutation on both sides of the dot product)
and makes the pairs (i, i + rot/2).

The reference has no such mixer (its attention keeps full keys and values per kv head,
core/src/model_executor/layers/attention.rs:91-231).
"""
from typing import Callable, Dict, Optional

import torch

from .base import (CacheBinding, CacheSpec, Mixer, Part, PartSpec, PositionEncoding, Runtime, TensorDecl, build_part,
                   register_part)
from .group_norm import GroupRMSNorm
from .linear import FusedLinear, Linear


class HeadMatrices(Part):
    """A checkpoint matrix [H * rows, cols] (head by head) kept as [H, rows, cols], or transposed per head as
    [H, cols, rows], for the per-head product kernel."""

    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, name: str, heads: int, rows: int, cols: int, transpose: bool):
        super().__init__(prefix, rt)
        self.name = "%s.%s" % (prefix, name)
        self.heads, self.rows, self.cols, self.transpose = int(heads), int(rows), int(cols), bool(transpose)
        self.weight: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        return {self.name: TensorDecl((self.heads * self.rows, self.cols))}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        w = fetch(self.name).reshape(self.heads, self.rows, self.cols)
        self.weight = (w.transpose(1, 2) if self.transpose else w).contiguous()


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int,
                 v_head_dim: int, kv_rank: int, q_rank: int, scale: float, eps: float, position: PartSpec,
                 owns_latent: bool = True, names: Optional[Dict[str, str]] = None, gate_per_entry: bool = False,
                 window: Optional[int] = None, cache_window: Optional[int] = None, weights_f32: bool = False):
        super().__init__(prefix, rt)
        self.gate_per_entry = bool(gate_per_entry)
        self.weights_f32 = bool(weights_f32)
        self.window = int(window) if window else None
        self.cache_window = int(cache_window) if cache_window else None
        if self.cache_window is not None and (self.window is None or self.window > self.cache_window):
            raise ValueError("%s: the pages are kept for %d positions, the layer's window is %r"
                             % (prefix, self.cache_window, self.window))
        self.H, self.dn, self.dr, self.dv = int(num_heads), int(head_dim), int(rot_dim), int(v_head_dim)
        self.R, self.Q = int(kv_rank), int(q_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.owns_latent = bool(owns_latent)
        # the cached row [c | r], padded with zeros to a width the matrix-core attention kernels take
        self.D = (self.R + self.dr + 15) // 16 * 16
        check = getattr(rt.ops, "check_head_dim", None)
        if check is not None:
            check(self.D, 1024)      # beyond 256 the general attention kernel serves it
        nm = dict(dq="dq", dkv="dkv", g="g", uq="uq", uk="uk", uv="uv", o="o", dq_norm="dq.norm", dkv_norm="dkv.norm")
        nm.update(names or {})
        # one product for everything that reads the layer's input: query latent, (key/value latent,) gates
        n_gate = self.H * self.dv if self.gate_per_entry else self.H
        sources = [(nm["dq"], self.Q)] + ([(nm["dkv"], self.R + self.dr)] if self.owns_latent else []) + [(nm["g"], n_gate)]
        # interleaved rotation pairs become pairs (i, i + rot/2) by the order of the rows that make them
        self.position: PositionEncoding = build_part("position", position, prefix, rt)
        rot = int(getattr(self.position, "rotary_dim", 0))
        tail = None
        if not getattr(self.position, "neox", True):
            if rot > self.dr:
                raise ValueError("%s: %d rotated entries in a part of %d" % (prefix, rot, self.dr))
            tail = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, self.dr))
        kv_order = None if tail is None else list(range(self.R)) + [self.R + i for i in tail]
        q_order = None if tail is None else [h * (self.dn + self.dr) + i for h in range(self.H)
                                             for i in list(range(self.dn)) + [self.dn + j for j in tail]]
        self.down = FusedLinear(prefix, rt, hidden_size, sources, bare_names=True,
                                row_orders={nm["dkv"]: kv_order} if (kv_order is not None and self.owns_latent) else None)
        self.at_kv = self.Q
        self.at_gate = self.Q + (self.R + self.dr if self.owns_latent else 0)
        self.q_norm = GroupRMSNorm("%s.%s" % (prefix, nm["dq_norm"]), rt, self.Q, self.eps, 1, weight_name="")
        self.kv_norm = GroupRMSNorm("%s.%s" % (prefix, nm["dkv_norm"]), rt, self.R, self.eps, 1, weight_name="") \
            if self.owns_latent else None
        self.uq = Linear(prefix, rt, nm["uq"], self.Q, self.H * (self.dn + self.dr), bare_names=True, row_order=q_order)
        self.uk_t = HeadMatrices(prefix, rt, nm["uk"], self.H, self.dn, self.R, transpose=True)     # [H, R, dn]
        self.uv = HeadMatrices(prefix, rt, nm["uv"], self.H, self.dv, self.R, transpose=False)      # [H, dv, R]
        self.o = Linear(prefix, rt, nm["o"], self.H * self.dv, hidden_size, bare_names=True)

    def children(self):
        return [p for p in (self.down, self.q_norm, self.kv_norm, self.uq, self.uk_t, self.uv, self.o, self.position)
                if p is not None]

    def cache_spec(self) -> Optional[CacheSpec]:
        return CacheSpec(num_kv_heads=1, head_dim=self.D, window=self.cache_window)

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        ops = self.rt.ops
        group = ctx.groups[binding.group]
        table, rot, _ = self.position.rotary_table()       # (interleaved pairs: see the order of the rows at load)
        table = table if rot == table.shape[1] else table[:, :rot]
        N = h.shape[0]
        low = self.down.forward(h)                                           # [N, Q (+ R + dr) + H]
        if binding.writes_cache:
            if not self.owns_latent:
                raise ValueError("%s has no latent of its own to store" % self.prefix)
            # the key/value latent into the pages and the query latent's norm, one launch
            cq = ops.latent_cache_write(low[:, self.at_kv:], self.kv_norm.weight, self.eps, self.R, self.dr, ctx.positions,
                                        table, group.slots, binding.k_pages, binding.v_pages,
                                        also_norm=low[:, :self.Q], also_weight=self.q_norm.weight)
        else:
            cq = self.q_norm.forward(low[:, :self.Q])
        q = self.uq.forward(cq)                                              # [N, H (dn + dr)]
        qa = torch.empty((N, self.H * self.D), dtype=q.dtype, device=q.device)
        # Uk_h^T qn_h -> qa[:, h, :R]; rotate(qr_h) -> qa[:, h, R:R + dr]; zeros behind
        ops.head_linear(q, self.dn + self.dr, self.uk_t.weight, qa, self.D,
                        rope_tail=(self.dn, self.R, self.dr, ctx.positions, table))
        more = {"weights_f32": True} if self.weights_f32 else {}
        a = ops.paged_attention(qa, binding.k_pages, binding.v_pages, group.block_tables, ctx.seg_of_token,
                                ctx.positions, self.H, 1, self.D, self.scale, self.window or 0, batch=ctx, **more)
        out = torch.empty((N, self.H * self.dv), dtype=q.dtype, device=q.device)
        ops.head_linear(a, self.D, self.uv.weight, out, self.dv, gate=low[:, self.at_gate:], gate_wide=self.gate_per_entry)
        return self.o.forward(out)
