"""Retention: linear attention with a fixed decay per head, no softmax and no denominator.

q = W_q h and k = W_k h (heads x dim), v = W_v h (heads x vdim); q and k are rotated by the position (optional; pairs
(i, i + rot/2) of the first ``rotary_dim`` entries); k is multiplied by ``key_scale`` (dim^-1/2 unless given). Per head
with decay g_h:   S_t = g_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t.
Every head's o is divided by its root mean square (no weight), the heads are multiplied by silu(W_g h) and projected by
W_o. The state of a request is S of every head, float32, in the engine's state slots: zeros when a request begins,
carried from step to step however the request is cut (csrc/retention.hip). The decays and everything behind the
projections are float32. The reference has no mixer with state (its only one is attention over a paged cache,
core/src/model_executor/layers/attention.rs:91-231).
"""
import math
from typing import Callable, Dict, Optional, Sequence

import torch

from .base import CacheBinding, Mixer, PartSpec, PositionEncoding, Runtime, StateSpec, build_part, register_part
from .linear import FusedLinear, Linear


@register_part("mixer", "retention")
class Retention(Mixer):
    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, heads: int, dim: int, vdim: int,
                 decay: Sequence[float], eps: float, position: Optional[PartSpec] = None,
                 key_scale: Optional[float] = None, names: Optional[Dict[str, str]] = None):
        super().__init__(prefix, rt)
        self.H, self.d, self.dv = int(heads), int(dim), int(vdim)
        self.eps = float(eps)
        self.decay_values = [float(g) for g in decay]
        if len(self.decay_values) != self.H or any(not (0.0 <= g <= 1.0) for g in self.decay_values):
            raise ValueError("%s: %d heads need %d decays within [0, 1], got %r" % (prefix, self.H, self.H, list(decay)))
        self.key_scale = float(key_scale) if key_scale is not None else self.d ** -0.5
        nm = dict(q="q", k="k", v="v", g="g", out="o")
        nm.update(names or {})
        H, d, dv = self.H, self.d, self.dv
        self.qkvg = FusedLinear(prefix, rt, hidden_size, [(nm["q"], H * d), (nm["k"], H * d), (nm["v"], H * dv),
                                                          (nm["g"], H * dv)], bare_names=True)
        self.o = Linear(prefix, rt, nm["out"], H * dv, hidden_size, bare_names=True)
        self.position: Optional[PositionEncoding] = build_part("position", position, prefix, rt) if position else None
        sizer = getattr(rt.ops, "retention_state_floats", None)
        self.state_floats = int(sizer(H, d, dv)) if sizer is not None else H * d * dv
        self.decay: Optional[torch.Tensor] = None

    def children(self):
        return [p for p in (self.qkvg, self.o, self.position) if p is not None]

    def tensors(self):
        return [self.decay] if self.decay is not None else []

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        # the decays and their logarithms, float32 (a decay of 0 forgets at once: a logarithm that is finite and
        # large stands for it, so that 0 times it is 0)
        logs = [max(math.log(g), -1e30) if g > 0.0 else -1e30 for g in self.decay_values]
        self.decay = torch.tensor(self.decay_values + logs, dtype=torch.float32).to(self.rt.device)

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.state_floats,), torch.float32)

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        H, d, dv = self.H, self.d, self.dv
        table = None
        if self.position is not None:
            rotary = self.position.rotary_table()
            if rotary is None or not rotary[2]:
                raise ValueError("%s rotates pairs (i, i + rot/2) from a table" % self.prefix)
            table = rotary[0]
        p = self.qkvg.forward(h)
        o = self.rt.ops.retention(p[:, :H * d], p[:, H * d:2 * H * d], p[:, 2 * H * d:2 * H * d + H * dv], self.decay,
                                  p[:, 2 * H * d + H * dv:], binding.state, ctx, H, d, dv, self.key_scale, self.eps,
                                  table=table)
        return self.o.forward(o)
