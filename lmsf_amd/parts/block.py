"""Arrangements of a layer's parts around the residual stream."""
from typing import Optional

import torch

from .base import Block, CacheBinding, Part, Runtime, TensorDecl, build_part, register_part
from .linear import Linear


@register_part("block", "prenorm_residual")
class PreNormResidualBlock(Block):
    """stream += mixer(norm_in(stream)); stream += ffn(norm_post(stream)).

    core/src/model_executor/models/llama/llama.rs:286-340. As there, an addition is carried out by
    the norm that follows it (vllm/kernels/layernorm_kernels.cu:41-68): the block receives the
    previous block's output not yet added, and returns its feed-forward output not yet added.
    Where the norm that follows accepts it, the o and down products may stay unfinished
    (``PendingProduct``) and the norm's kernel adds up their partial sums; where a norm may defer
    its work and the part after it takes that, the norm runs inside that part's first product.
    A layer without a feed-forward (a part that says ``absent``) has only the first sublayer and needs no
    "post_mixer" norm: the mixer's output is what the block returns, not yet added.
    """

    graph_safe = True

    ROLES = ("input",)          # and "post_mixer" where there is a feed-forward

    def __init__(self, prefix: str, rt, mixer, feed_forward, norms):
        super().__init__(prefix, rt, mixer, feed_forward, norms)
        self.has_ffn = not getattr(feed_forward, "absent", False)
        if self.has_ffn and "post_mixer" not in norms:
            raise ValueError("block %s needs norms post_mixer (before its feed-forward)" % type(self).__name__)

    @property
    def accepts_pending_branch(self) -> bool:
        return self.norms["input"].accepts_pending

    def forward(self, branch: Optional[torch.Tensor], residual: torch.Tensor, ctx,
                binding: CacheBinding) -> torch.Tensor:
        first, post = self.norms["input"], self.norms.get("post_mixer")
        if first.may_defer and self.mixer.accepts_normed:
            h = first.forward_add(branch, residual, defer_ok=True)
        else:
            h = first.forward_add(branch, residual)
        if not self.has_ffn:
            if self.mixer.may_return_pending and self.pending_output_ok:
                return self.mixer.forward(h, ctx, binding, pending_ok=True)
            return self.mixer.forward(h, ctx, binding)
        if self.mixer.may_return_pending and post.accepts_pending:
            a = self.mixer.forward(h, ctx, binding, pending_ok=True)
        else:
            a = self.mixer.forward(h, ctx, binding)
        if post.may_defer and self.feed_forward.accepts_normed:
            h = post.forward_add(a, residual, defer_ok=True)
        else:
            h = post.forward_add(a, residual)
        if self.feed_forward.may_return_pending and self.pending_output_ok:
            return self.feed_forward.forward(h, pending_ok=True)
        return self.feed_forward.forward(h)


@register_part("block", "sandwich_depth_average")
class SandwichDepthBlock(Block):
    """A norm before and after each sublayer, and a weighted average over depth:

        x += norm_b(mixer(norm_a(x)));   x += norm_d(ffn(norm_c(x)));   X_k = x;   x = sum_j<=k mix[j] X_j

    with X_0 the embedding's output and X_k the result of the k-th layer run (k = ``depth``), before the
    averaging. The stream and every X_j are float32. The results lie in one buffer [depth_total + 1, N, W] that
    the first block of a step allocates and the others find in ``ctx.aux``. The addition after the mixer and the
    norm before the feed-forward are one kernel; so are the addition after the feed-forward, the storing of
    X_k, the averaging and (where the model has linked the blocks) the first norm of the block that follows.
    Nothing is left to add when the block returns.

    The reference's only arrangement is the pre-norm one above (core/src/model_executor/models/llama/llama.rs:286-340).
    """

    graph_safe = True
    recordable = False

    ROLES = ("pre_mixer", "post_mixer")          # "pre_ffn" and "post_ffn" too where there is a feed-forward

    def __init__(self, prefix: str, rt: Runtime, mixer, feed_forward, norms, depth: int, depth_total: int,
                 mix=None):
        super().__init__(prefix, rt, mixer, feed_forward, norms)
        self.depth, self.depth_total = int(depth), int(depth_total)
        if not (1 <= self.depth <= self.depth_total):
            raise ValueError("block %s: depth %d of %d" % (prefix, self.depth, self.depth_total))
        self.has_ffn = not getattr(feed_forward, "absent", False)
        if self.has_ffn and not ("pre_ffn" in norms and "post_ffn" in norms):
            raise ValueError("block %s needs the norms pre_ffn and post_ffn around its feed-forward" % prefix)
        self.mix = build_part("norm", mix, prefix, rt) if mix is not None else None
        self._ffn_takes_ids = bool(getattr(feed_forward, "needs_token_ids", False))
        self.next_norm = None       # the norm that the block after this one begins with, where the model has linked it

    def link_next(self, following: Block) -> None:
        """The model tells a block which block always runs after it: this one's last kernel then also computes that
        one's first norm (one launch a layer less) and leaves it in ``ctx.aux["prenormed"]``."""
        if isinstance(following, SandwichDepthBlock):
            self.next_norm = following.norms["pre_mixer"]

    def children(self):
        return super().children() + ([self.mix] if self.mix is not None else [])

    def forward(self, branch: Optional[torch.Tensor], residual: torch.Tensor, ctx, binding: CacheBinding):
        if branch is not None:
            raise ValueError("sandwich_depth_average takes no branch that is still to be added")
        n = self.norms
        hist = ctx.aux.get("depth_history")
        if self.depth == 1 or hist is None or hist.shape[1:] != residual.shape:
            hist = torch.empty((self.depth_total + 1,) + tuple(residual.shape), dtype=torch.float32,
                               device=residual.device)
            hist[0].copy_(residual)
            ctx.aux["depth_history"] = hist
        mix = self.mix.weight if self.mix is not None else None
        h = ctx.aux.pop("prenormed", None)
        if h is None:
            h = n["pre_mixer"].forward(residual)
        a = self.mixer.forward(h, ctx, binding)
        if not self.has_ffn:
            self._close(n["post_mixer"], a, residual, hist, mix, ctx)
            return None
        h = n["post_mixer"].add_normed(a, residual, then=n["pre_ffn"])
        f = self.feed_forward.forward(h, token_ids=ctx.token_ids) if self._ffn_takes_ids else self.feed_forward.forward(h)
        self._close(n["post_ffn"], f, residual, hist, mix, ctx)
        return None

    def _close(self, norm, branch, residual, hist, mix, ctx) -> None:
        if mix is None:
            ahead = norm.add_normed(branch, residual, then=self.next_norm)
            hist[self.depth].copy_(residual)
        else:
            ahead = norm.add_normed(branch, residual, then=self.next_norm, history=hist, index=self.depth, mix=mix)
        if ahead is not None:
            ctx.aux["prenormed"] = ahead


@register_part("block", "parallel_scaled")
class ParallelScaledBlock(Block):
    """One norm, two sublayers that both read it, each result scaled entry by entry before the sum:

        h = norm(x);   x += scale_mixer * mixer(h) + scale_ffn * ffn(h)

    (without a feed-forward only the first term). The scales are checkpoint vectors of the layer, float32, as are
    the stream and the sum. The addition and the norm that the next block begins with are one kernel where the
    model has linked the blocks (``link_next``); nothing is left to add when the block returns. The reference's
    only arrangement is the pre-norm one with two norms (core/src/model_executor/models/llama/llama.rs:286-340).
    """

    graph_safe = True
    recordable = False

    ROLES = ("input",)

    def __init__(self, prefix: str, rt: Runtime, mixer, feed_forward, norms, hidden_size: int,
                 mixer_scale_name: str = "ls1", ffn_scale_name: str = "ls2"):
        super().__init__(prefix, rt, mixer, feed_forward, norms)
        self.has_ffn = not getattr(feed_forward, "absent", False)
        self.W = int(hidden_size)
        self.names = ("%s.%s" % (prefix, mixer_scale_name), "%s.%s" % (prefix, ffn_scale_name))
        self.mixer_scale: Optional[torch.Tensor] = None
        self.ffn_scale: Optional[torch.Tensor] = None
        self.next_norm = None

    def link_next(self, following: Block) -> None:
        """The block that always runs after this one begins with a norm of the stream: this block's closing kernel
        computes it as well and leaves it in ``ctx.aux["prenormed"]``."""
        nxt = following.norms.get("input") if isinstance(following, ParallelScaledBlock) else None
        if nxt is not None and getattr(nxt, "weight_offset", 0.0) == 0.0 and hasattr(nxt, "eps"):
            self.next_norm = nxt

    def checkpoint_tensors(self):
        from .base import TensorDecl
        out = {self.names[0]: TensorDecl((self.W,), init="ones", keeps_float32=True)}
        if self.has_ffn:
            out[self.names[1]] = TensorDecl((self.W,), init="ones", keeps_float32=True)
        return out

    def load_weights(self, fetch) -> None:
        self.mixer_scale = fetch(self.names[0]).to(torch.float32).contiguous()
        if self.has_ffn:
            self.ffn_scale = fetch(self.names[1]).to(torch.float32).contiguous()

    def tensors(self):
        return [t for t in (self.mixer_scale, self.ffn_scale) if t is not None]

    def forward(self, branch: Optional[torch.Tensor], residual: torch.Tensor, ctx, binding: CacheBinding):
        norm = self.norms["input"]
        h = ctx.aux.pop("prenormed", None) if branch is None else None
        if h is None:
            h = norm.forward_add(branch, residual)
        a = self.mixer.forward(h, ctx, binding)
        f = self.feed_forward.forward(h) if self.has_ffn else None
        nxt = self.next_norm
        ahead = self.rt.ops.scale_add_norm(a, self.mixer_scale, f, self.ffn_scale, residual,
                                           weight=nxt.weight if nxt is not None else None,
                                           eps=nxt.eps if nxt is not None else 0.0)
        if ahead is not None:
            ctx.aux["prenormed"] = ahead
        return None


class StreamInjection(Part):
    """x <- M [x ; x0]: the stream and the embedding's output side by side through one matrix [W, 2 W] (the stream's
    columns first). The product's operands are in the run's type, its result and the stream float32."""

    graph_safe = True
    recordable = False

    def __init__(self, name: str, rt: Runtime, hidden_size: int):
        super().__init__(name, rt)
        self.W = int(hidden_size)
        self.proj = Linear("", rt, name, 2 * self.W, self.W, bare_names=True)

    def children(self):
        return [self.proj]

    def forward(self, residual: torch.Tensor, ctx) -> None:
        x0 = ctx.aux.get("embedding_output")
        if x0 is None:
            raise ValueError("%s: the embedding did not keep its output for this step" % self.prefix)
        ops = self.rt.ops
        both = ops.concat_rows(residual, x0, self.rt.dtype)
        ops.linear_wide(both, self.proj.weight, None, out=residual)       # (the operand is the copy just made)


class TokenSideInput(Part):
    """A per-layer input from the token itself, added to the stream: e = a slice of the token's row of a table shared
    by the layers; g = gelu_tanh(W_gate x) * e; y = W_proj g; x += y / rms(y) * w (a plain RMS-norm weight)."""

    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, dim: int, at: int, table_name: str, table_width: int,
                 vocab_size: int, eps: float, gate_name: str = "gate", proj_name: str = "proj", norm_name: str = "norm"):
        super().__init__(prefix, rt)
        self.W, self.dim, self.at, self.eps = int(hidden_size), int(dim), int(at), float(eps)
        self.table_name, self.table_shape = str(table_name), (int(vocab_size), int(table_width))
        if not (0 <= self.at and self.at + self.dim <= self.table_shape[1]):
            raise ValueError("%s: entries %d to %d of a table row of %d" % (prefix, at, at + dim, table_width))
        self.gate = Linear(prefix, rt, gate_name, self.W, self.dim, bare_names=True)
        self.proj = Linear(prefix, rt, proj_name, self.dim, self.W, bare_names=True)
        self.norm_name = "%s.%s" % (prefix, norm_name)
        self.table: Optional[torch.Tensor] = None
        self.norm_weight: Optional[torch.Tensor] = None

    def children(self):
        return [self.gate, self.proj]

    def checkpoint_tensors(self):
        return {self.table_name: TensorDecl(self.table_shape),
                self.norm_name: TensorDecl((self.W,), init="ones", keeps_float32=True)}

    def load_weights(self, fetch) -> None:
        self.table = fetch(self.table_name).contiguous()            # (one device tensor for all layers: the loader shares it)
        self.norm_weight = fetch(self.norm_name).to(torch.float32).contiguous()

    def tensors(self):
        return [t for t in (self.norm_weight,) if t is not None]

    def forward(self, residual: torch.Tensor, ctx, x: Optional[torch.Tensor] = None, then=None) -> Optional[torch.Tensor]:
        """``x``: the stream in the run's type, where the caller has it already. ``then``: a norm of the new stream
        that the closing kernel computes as well; its result is returned."""
        ops = self.rt.ops
        if x is None:
            x = ops.group_norm(residual=residual, out_dtype=self.rt.dtype)      # the stream in the run's type
        g = ops.gate_table(self.gate.forward(x), ctx.token_ids, self.table, self.at)
        y = ops.linear_wide(g, self.proj.weight, None)
        return ops.group_norm(x=y, x_weight=self.norm_weight, residual=residual, x_eps=self.eps,
                              out_weight=then.weight if then is not None else None,
                              out_eps=then.eps if then is not None else self.eps, out_dtype=self.rt.dtype,
                              want_out=then is not None)


@register_part("block", "sandwich")
class SandwichBlock(Block):
    """A norm before and after each sublayer:

        x += norm_b(mixer(norm_a(x)));   x += norm_d(ffn(norm_c(x)))

    (without a feed-forward only the first), optionally with the stream replaced by a product over the stream and the
    embedding's output before the block (``inject``: the name of the matrix; a block that begins a pass of a loop over
    layers) and a per-layer input from the token added after it (``side``: the parameters of ``TokenSideInput``). The
    stream is float32; nothing is left to add when the block returns. The addition after the mixer and the norm
    before the feed-forward are one kernel; the addition after the feed-forward also hands the side input the stream in
    the run's type; and the block's last kernel also computes the first norm of the block that always follows, where
    that block does not replace the stream first (``link_next``). The reference's only arrangement is the pre-norm one
    (core/src/model_executor/models/llama/llama.rs:286-340)."""

    graph_safe = True
    recordable = False

    ROLES = ("pre_mixer", "post_mixer")          # "pre_ffn" and "post_ffn" too where there is a feed-forward

    def __init__(self, prefix: str, rt: Runtime, mixer, feed_forward, norms, hidden_size: int,
                 inject: Optional[str] = None, side=None):
        super().__init__(prefix, rt, mixer, feed_forward, norms)
        self.has_ffn = not getattr(feed_forward, "absent", False)
        if self.has_ffn and not ("pre_ffn" in norms and "post_ffn" in norms):
            raise ValueError("block %s needs the norms pre_ffn and post_ffn around its feed-forward" % prefix)
        self.inject = StreamInjection(inject, rt, hidden_size) if inject else None
        self.side = TokenSideInput("%s.%s" % (prefix, dict(side).pop("prefix", "side")), rt, hidden_size=hidden_size,
                                   **{k: v for k, v in dict(side).items() if k != "prefix"}) if side else None
        self._ffn_takes_ids = bool(getattr(feed_forward, "needs_token_ids", False))
        self.next_norm = None       # the norm that the block after this one begins with, where the model has linked it

    def link_next(self, following: Block) -> None:
        """The model tells a block which block always runs after it: this one's last kernel then also computes that
        one's first norm and leaves it in ``ctx.aux["prenormed"]``. Not where the following block replaces the stream
        before its norm."""
        if not isinstance(following, SandwichBlock) or following.inject is not None:
            return
        nxt = following.norms["pre_mixer"]
        # (one kernel takes one number of groups for both of its norms: the side input's norm has one group, a
        # block without side input closes with its own last norm)
        closing = 1 if self.side is not None else self.norms["post_ffn" if self.has_ffn else "post_mixer"].groups
        if getattr(nxt, "groups", None) == closing:
            self.next_norm = nxt

    def children(self):
        return super().children() + [p for p in (self.inject, self.side) if p is not None]

    def _close(self, norm, branch: torch.Tensor, residual: torch.Tensor, ctx) -> None:
        """stream += norm(branch), then the side input; the last of these kernels also computes the next block's norm."""
        ops = self.rt.ops
        if self.side is None:
            ahead = norm.add_normed(branch, residual, then=self.next_norm)
        else:
            # (no weight behind the sum: the kernel hands back the new stream itself, in the run's type)
            x = ops.group_norm(x=branch, x_weight=norm.weight, residual=residual, groups=norm.groups, x_eps=norm.eps,
                               out_dtype=self.rt.dtype)
            ahead = self.side.forward(residual, ctx, x=x, then=self.next_norm)
        if ahead is not None:
            ctx.aux["prenormed"] = ahead

    def forward(self, branch: Optional[torch.Tensor], residual: torch.Tensor, ctx, binding: CacheBinding):
        if branch is not None:
            raise ValueError("sandwich takes no branch that is still to be added")
        n = self.norms
        h = ctx.aux.pop("prenormed", None)
        if self.inject is not None:
            self.inject.forward(residual, ctx)
            h = None
        if h is None:
            h = n["pre_mixer"].forward(residual)
        a = self.mixer.forward(h, ctx, binding)
        if self.has_ffn:
            h = n["post_mixer"].add_normed(a, residual, then=n["pre_ffn"])
            f = self.feed_forward.forward(h, token_ids=ctx.token_ids) if self._ffn_takes_ids else self.feed_forward.forward(h)
            self._close(n["post_ffn"], f, residual, ctx)
        else:
            self._close(n["post_mixer"], a, residual, ctx)
        return None
