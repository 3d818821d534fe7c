"""RMS norm in groups, and the weights of a running average over the layers' results.

gn(v; w)_i = v_i / sqrt(mean over i's part of v^2 + eps) * w_i, the row cut into ``groups`` equal consecutive
parts; groups = 1 is the plain RMS norm. All arithmetic is float32 (csrc/group_norm.hip). The reference's
norm is the single-group case (vllm/kernels/layernorm_kernels.cu:13-38); it has no norm after a sublayer
and no averaging over depth.
"""
from typing import Callable, Dict, Optional

import torch

from .base import Norm, Part, Runtime, TensorDecl, register_part


@register_part("norm", "group_rms_norm")
class GroupRMSNorm(Norm):
    """``weight_name`` is appended to the prefix with a dot ("" : the tensor is the prefix itself). ``weight_offset``
    is added to the stored weight at load (1 for a weight that is stored around zero and acts as 1 + w)."""

    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, size: int, eps: float, groups: int = 1, weight_name: str = "weight",
                 weight_offset: float = 0.0):
        super().__init__(prefix, rt)
        self.size, self.eps, self.groups = int(size), float(eps), int(groups)
        self.weight_offset = float(weight_offset)
        if self.groups <= 0 or self.size % self.groups:
            raise ValueError("norm %r: %d columns do not split into %d groups" % (prefix, self.size, self.groups))
        self.weight_name = "%s.%s" % (prefix, weight_name) if weight_name else prefix
        self.weight: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        init = "ones" if self.weight_offset == 0.0 else "zeros"
        return {self.weight_name: TensorDecl((self.size,), init=init, keeps_float32=True)}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        w = fetch(self.weight_name).to(torch.float32)
        self.weight = (w + self.weight_offset if self.weight_offset != 0.0 else w).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """gn of a float32 stream (or of activations, also a view with unit column stride) in the run's dtype."""
        if x.dtype == torch.float32 and x.is_contiguous():
            return self.rt.ops.group_norm(residual=x, out_weight=self.weight, groups=self.groups, out_eps=self.eps,
                                          out_dtype=self.rt.dtype)
        return self.rt.ops.group_norm(x=x, x_weight=self.weight, groups=self.groups, x_eps=self.eps,
                                      out_dtype=self.rt.dtype)

    def forward_add(self, branch: Optional[torch.Tensor], residual: torch.Tensor,
                    rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """gn(residual) at ``rows``; this norm adds nothing to the stream (a branch is added by ``add_normed`` of
        the norm that follows the sublayer)."""
        if branch is not None:
            raise ValueError("group_rms_norm takes no branch to add before it")
        return self.rt.ops.group_norm(residual=residual, out_weight=self.weight, groups=self.groups, out_eps=self.eps,
                                      out_dtype=self.rt.dtype, rows=rows)

    def add_normed(self, branch: torch.Tensor, residual: torch.Tensor, then: Optional["GroupRMSNorm"] = None,
                   history: Optional[torch.Tensor] = None, index: int = 0,
                   mix: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """residual += gn(branch), in float32 and in place. With ``history`` the sum is stored as result number
        ``index`` and the stream becomes sum_j mix[j] history[j]. With ``then`` (the norm before the next
        sublayer) returns that norm of the new stream, from the same kernel."""
        return self.rt.ops.group_norm(
            x=branch, x_weight=self.weight, residual=residual, out_weight=then.weight if then is not None else None,
            groups=self.groups, x_eps=self.eps, out_eps=then.eps if then is not None else self.eps,
            out_dtype=self.rt.dtype, history=history, index=index, mix=mix, want_out=then is not None)


@register_part("norm", "depth_mix")
class DepthMix(Part):
    """The weights of the average over the results of the layers so far: one per result, float32."""

    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, count: int, weight_name: str = "dwa"):
        super().__init__(prefix, rt)
        self.count = int(count)
        self.weight_name = "%s.%s" % (prefix, weight_name)
        self.weight: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        return {self.weight_name: TensorDecl((self.count,), init="last_one", keeps_float32=True)}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).to(torch.float32).contiguous()
