"""Softmax attention over the paged cache with norms on the whole projections, rotated values and bounded scores.

H query heads and G key/value heads (query head h uses key/value head h // (H / G)), ``dim`` entries a query or key,
``vdim`` a value. In the order in which they act:

- q = W_q h, k = W_k h, v = W_v h, no biases;
- one RMS norm over all H dim entries of q and one over all G dim entries of k, each with a weight of that size
  (``qk_norm``), before the heads are split and before rotation;
- rotary positions on the first ``rotary_dim`` entries of every q and k head;
- every value head divided by its root mean square, no weight (``value_norm``);
- the value of position j turned by j over all vdim entries (``value_position``: a rotation over vdim), cached so;
- score = q . k * scale, then cap tanh(score / cap) (``softcap``); causal, within a window of the last positions;
- every head's sum over the values turned back by the query's position (so that a value enters turned by j - i);
- head h times sigmoid(W_g h)_h, one number a head (``head_gate``), then W_o.

Pairs of a rotation are (2m, 2m + 1) or (m, m + n/2) as the position parts say (both must say the same). The
attention kernels take one head size: keys and values are cached padded with zeros to D = max(dim, vdim) rounded up
to 16. Keys and values are written to the pages before any query reads, so every way of cutting a request into steps
is one case. The reference's attention has none of the extras (core/src/model_executor/layers/attention.rs:91-231).
"""
from typing import Callable, Dict, Optional

import torch

from .base import (CacheBinding, CacheSpec, Mixer, PartSpec, PositionEncoding, Runtime, TensorDecl, build_part,
                   register_part)
from .linear import FusedLinear, Linear


@register_part("mixer", "normed_attention")
class NormedAttention(Mixer):
    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 v_head_dim: int, scale: float, eps: float, position: Optional[PartSpec] = None,
                 value_position: Optional[PartSpec] = None, qk_norm: bool = True, value_norm: bool = True,
                 softcap: float = 0.0, window: Optional[int] = None, head_gate: bool = True,
                 names: Optional[Dict[str, str]] = None):
        super().__init__(prefix, rt)
        self.H, self.G, self.dim, self.vdim = int(num_heads), int(num_kv_heads), int(head_dim), int(v_head_dim)
        if self.H % self.G:
            raise ValueError("%s: heads %d is not a multiple of kv_heads %d" % (prefix, self.H, self.G))
        if self.dim % 2 or self.vdim % 2:
            raise ValueError("%s: key and value sizes must be even, are %d and %d" % (prefix, self.dim, self.vdim))
        self.scale, self.eps, self.softcap = float(scale), float(eps), float(softcap or 0.0)
        if not self.scale > 0 or self.softcap < 0:
            raise ValueError("%s: the scale must be positive and the soft cap not negative" % prefix)
        self.window = int(window) if window else None
        self.qk_norm, self.value_norm, self.has_gate = bool(qk_norm), bool(value_norm), bool(head_gate)
        self.D = (max(self.dim, self.vdim) + 15) // 16 * 16
        check = getattr(rt.ops, "check_head_dim", None)
        if check is not None:
            check(self.D, 1024)
        nm = dict(q="q", k="k", v="v", g="g", o="o", q_norm="q.norm", k_norm="k.norm")
        nm.update(names or {})
        self.nm = nm
        H, G = self.H, self.G
        self.n_qkv = (H + G) * self.dim + G * self.vdim
        sources = [(nm["q"], H * self.dim), (nm["k"], G * self.dim), (nm["v"], G * self.vdim)]
        if self.has_gate:
            sources.append((nm["g"], H))
        self.proj = FusedLinear(prefix, rt, hidden_size, sources, bare_names=True, pad_rows_to=8)
        self.o = Linear(prefix, rt, nm["o"], H * self.vdim, hidden_size, bare_names=True)
        self.position: Optional[PositionEncoding] = build_part("position", position, prefix, rt) if position else None
        self.value_position: Optional[PositionEncoding] = build_part("position", value_position, prefix, rt) \
            if value_position else None
        self.q_weight: Optional[torch.Tensor] = None
        self.k_weight: Optional[torch.Tensor] = None

    def children(self):
        return [p for p in (self.proj, self.o, self.position, self.value_position) if p is not None]

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        if not self.qk_norm:
            return {}
        return {"%s.%s" % (self.prefix, self.nm["q_norm"]): TensorDecl((self.H * self.dim,), init="ones", keeps_float32=True),
                "%s.%s" % (self.prefix, self.nm["k_norm"]): TensorDecl((self.G * self.dim,), init="ones", keeps_float32=True)}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        if self.qk_norm:
            self.q_weight = fetch("%s.%s" % (self.prefix, self.nm["q_norm"])).to(torch.float32).contiguous()
            self.k_weight = fetch("%s.%s" % (self.prefix, self.nm["k_norm"])).to(torch.float32).contiguous()

    def tensors(self):
        return [t for t in (self.q_weight, self.k_weight) if t is not None]

    def cache_spec(self) -> Optional[CacheSpec]:
        return CacheSpec(num_kv_heads=self.G, head_dim=self.D, window=self.window)

    def _tables(self):
        table = table_v = None
        styles = set()
        if self.position is not None:
            table, _, neox = self.position.rotary_table()
            styles.add(bool(neox))
        if self.value_position is not None:
            table_v, rot_v, neox = self.value_position.rotary_table()
            if rot_v != self.vdim:
                raise ValueError("%s: values are rotated over all their %d entries" % (self.prefix, self.vdim))
            styles.add(bool(neox))
        if len(styles) > 1:
            raise ValueError("%s: keys and values must pair their entries alike" % self.prefix)
        return table, table_v, (not styles.pop()) if styles else False

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        ops = self.rt.ops
        H, G, dim, vdim, D = self.H, self.G, self.dim, self.vdim, self.D
        group = ctx.groups[binding.group]
        table, table_v, interleaved = self._tables()
        p = self.proj.forward(h)                                   # [N, q | k | v (| g) | padding]
        q, k, v = p[:, :H * dim], p[:, H * dim:(H + G) * dim], p[:, (H + G) * dim:self.n_qkv]
        slots = group.slots if binding.writes_cache else None
        qa = ops.attn_prepare_normed(q, k, v, H, G, dim, vdim, D, ctx.positions, slots, binding.k_pages, binding.v_pages,
                                     q_weight=self.q_weight, k_weight=self.k_weight, eps=self.eps, table=table,
                                     table_v=table_v, interleaved=interleaved, v_norm=self.value_norm)
        a = ops.paged_attention(qa, binding.k_pages, binding.v_pages, group.block_tables, ctx.seg_of_token,
                                ctx.positions, H, G, D, self.scale, self.window or 0, batch=ctx, softcap=self.softcap)
        a = ops.attn_finish(a, D, H, vdim, ctx.positions, gate=p[:, self.n_qkv:] if self.has_gate else None,
                            table_v=table_v, interleaved=interleaved)
        return self.o.forward(a)
