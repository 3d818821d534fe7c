"""The gated delta rule with a decay per head and key channel: a matrix memory of fixed size per request.

q = W_q h and k = W_k h (G heads of ``dim``), v = W_v h (H heads of ``vdim``; head h reads q/k head h // (H / G)); each
passes a short causal convolution over time per channel and SiLU; q and k are made unit vectors per head,
x / sqrt(sum x^2 + 1e-6), q also times dim^-1/2. beta = sigmoid(W_b h), one per head. One decay per head and key
channel, g = exp(-exp(A_log_h) softplus(W_a2 (W_a1 h) + dt_bias)). Per head, token by token:

    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

(the read-out sees the token's own write). Every head's o over its root mean square, times a weight over vdim shared
by the heads, times sigmoid(W_g2 (W_g1 h)); then W_o. A request's state: S [H, dim, vdim] float32 and the
convolutions' last taps - 1 inputs. What enters the recurrence beside the projections and the convolutions (unit
norms, beta, the decays with their softplus and exponentials, S) is float32 (csrc/delta_rule.hip). The reference has no
mixer with state (core/src/model_executor/layers/attention.rs:91-231 is its only mixer).
"""
from typing import Dict, Optional

import torch

from .base import CacheBinding, Mixer, Runtime, StateSpec, register_part
from .linear import FusedLinear, Linear
from .recurrent import FloatVector, ShortConv


@register_part("mixer", "gated_delta")
class GatedDelta(Mixer):
    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int,
                 conv: int, decay_rank: int, gate_rank: int, eps: float, unit_eps: float = 1e-6,
                 names: Optional[Dict[str, str]] = None):
        super().__init__(prefix, rt)
        self.H, self.G, self.d, self.dv, self.taps = int(heads), int(kv_heads), int(dim), int(vdim), int(conv)
        if self.H % self.G:
            raise ValueError("%s: heads %d is not a multiple of kv_heads %d" % (prefix, self.H, self.G))
        if self.d > 256:
            raise ValueError("%s: keys of %d entries (at most 256)" % (prefix, self.d))
        self.eps, self.unit_eps = float(eps), float(unit_eps)
        self.ra, self.rg = int(decay_rank), int(gate_rank)
        nm = dict(q="q", k="k", v="v", conv="conv", b="b", a1="a1", a2="a2", dt_bias="dt_bias", a_log="A_log", g1="g1",
                  g2="g2", norm="norm", out="o")
        nm.update(names or {})
        H, G, d, dv = self.H, self.G, self.d, self.dv
        self.n_qkv = 2 * G * d + H * dv
        # one product for everything that reads the layer's input and may be rounded: q | k | v | a1 | g1
        self.proj = FusedLinear(prefix, rt, hidden_size, [(nm["q"], G * d), (nm["k"], G * d), (nm["v"], H * dv),
                                                          (nm["a1"], self.ra), (nm["g1"], self.rg)], bare_names=True,
                                pad_rows_to=8)
        self.beta = FusedLinear(prefix, rt, hidden_size, [(nm["b"], H)], bare_names=True, pad_rows_to=8)
        self.conv = ShortConv(prefix, rt, [("%s.%s" % (nm[x], nm["conv"]), n) for x, n in
                                           (("q", G * d), ("k", G * d), ("v", H * dv))], self.taps, activation="silu")
        self.a2 = FusedLinear(prefix, rt, self.ra, [(nm["a2"], H * d)], bare_names=True, pad_rows_to=8)
        self.g2 = Linear(prefix, rt, nm["g2"], self.rg, H * dv, bare_names=True)
        self.dt_bias = FloatVector("%s.%s" % (prefix, nm["dt_bias"]), rt, (H * d,), init="zeros")
        self.a_log = FloatVector("%s.%s" % (prefix, nm["a_log"]), rt, (H,), init="const:0.0")
        self.norm = FloatVector("%s.%s" % (prefix, nm["norm"]), rt, (dv,), init="ones")
        self.o = Linear(prefix, rt, nm["out"], H * dv, hidden_size, bare_names=True)
        sizer = getattr(rt.ops, "gated_delta_state_floats", None)
        self.memory_floats = int(sizer(H, d, dv)) if sizer is not None else H * d * dv

    def children(self):
        return [self.proj, self.beta, self.conv, self.a2, self.g2, self.dt_bias, self.a_log, self.norm, self.o]

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.memory_floats + self.conv.state_floats,), torch.float32)

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        ops = self.rt.ops
        H, G, d, dv = self.H, self.G, self.d, self.dv
        st = binding.state
        p = self.proj.forward(h)                                              # [N, q | k | v | a1 | g1 | padding]
        qkv = self.conv.forward(p[:, :self.n_qkv], ctx, st[:, self.memory_floats:] if self.taps > 1 else None)
        a1 = p[:, self.n_qkv:self.n_qkv + self.ra]
        g1 = p[:, self.n_qkv + self.ra:self.n_qkv + self.ra + self.rg]
        a = ops.linear_wide(a1, self.a2.weight, None)                         # float32: it enters the decay
        b = ops.linear_wide(h, self.beta.weight, None)                        # float32: beta before its sigmoid
        gate = self.g2.forward(g1)
        raw = ops.gated_delta(qkv, 0, G * d, 2 * G * d, a, self.dt_bias.weight, self.a_log.weight, b, st, ctx, H, G, d,
                              dv, d ** -0.5, self.unit_eps)
        o = ops.head_rms_gate(raw, H, dv, self.eps, self.norm.weight, gate, self.rt.dtype, "sigmoid")
        return self.o.forward(o)
