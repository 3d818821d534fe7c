"""Token embedding and the LM head.

Embedding: a row gather of the [V, H] table (core/src/model_executor/layers/vocab_parallel_embedding.rs:28-38),
written as the float32 residual stream, optionally scaled (Gemma multiplies by sqrt(H),
core/src/model_executor/models/gemma/gemma.rs:244). Head: logits = h W^T in float32
(core/src/model_executor/models/llama/llama.rs:471); with tied embeddings the head's matrix is the
embedding table (the reference parses tie_word_embeddings and ignores it, llama.rs:487-492).
"""
from typing import Callable, Dict, Optional

import torch

from .base import Part, Runtime, StateSpec, TensorDecl, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, vocab_size: int, hidden_size: int, scale: float = 1.0,
                 weight_name: str = "weight"):
        super().__init__(prefix, rt)
        self.vocab_size, self.hidden_size, self.scale = int(vocab_size), int(hidden_size), float(scale)
        # (weight_name "": the table is the tensor ``prefix`` itself)
        self.weight_name = "%s.%s" % (prefix, weight_name) if weight_name else prefix
        self.weight: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        return {self.weight_name: TensorDecl((self.vocab_size, self.hidden_size))}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).contiguous()

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        """int32 [N] -> float32 [N, H]."""
        return self.rt.ops.embedding(token_ids, self.weight, self.scale)


@register_part("embedding", "hashed_pair_embedding")
class HashedPairEmbedding(Part):
    """x = table[id] + pairs[row]: beside the token's own row a row of a second table chosen by a hash of the token
    before it and the token, row = (previous id * mul_prev + id * mul_cur) mod buckets; a request's first token takes
    the table's last row (number ``buckets``). The sum is float32. The token before a step's first token is part of
    the request's state: one int32 per state slot (``state_spec``; the engine hands the tensor over through
    ``bind_state``), written by the kernel that reads it. ``keep_output``: the result is also left in
    ``ctx.aux["embedding_output"]`` for parts that read it after the stream has moved on. The reference's embedding is
    the plain row gather (core/src/model_executor/layers/vocab_parallel_embedding.rs:28-38)."""

    graph_safe = True
    recordable = False
    needs_context = True            # the model calls forward_step(ctx) instead of forward(token_ids)

    def __init__(self, prefix: str, rt: Runtime, vocab_size: int, hidden_size: int, buckets: int, mul_prev: int,
                 mul_cur: int, pair_name: str = "bigram", weight_name: str = "", keep_output: bool = False):
        super().__init__(prefix, rt)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        if self.buckets < 1 or self.mul_prev < 0 or self.mul_cur < 0:
            raise ValueError("hashed_pair_embedding: buckets must be > 0 and the multipliers >= 0")
        self.weight_name = "%s.%s" % (prefix, weight_name) if weight_name else prefix
        self.pair_name = str(pair_name)
        self.keep_output = bool(keep_output)
        self.weight: Optional[torch.Tensor] = None
        self.pairs: Optional[torch.Tensor] = None
        self.prev_state: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        return {self.weight_name: TensorDecl((self.vocab_size, self.hidden_size)),
                self.pair_name: TensorDecl((self.buckets + 1, self.hidden_size))}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).contiguous()
        self.pairs = fetch(self.pair_name).to(self.weight.dtype).contiguous()

    def tensors(self):
        return [t for t in (self.weight, self.pairs) if t is not None]

    def state_spec(self) -> StateSpec:
        return StateSpec((1,), torch.int32)

    def bind_state(self, state: torch.Tensor) -> None:
        self.prev_state = state.view(-1)

    def forward_step(self, ctx) -> torch.Tensor:
        """The step's tokens -> float32 [N, H]."""
        if self.prev_state is None:
            raise ValueError("hashed_pair_embedding: no state was bound (the token before a step's first)")
        if not self.keep_output:
            return self.rt.ops.hashed_pair_embedding(ctx, self.weight, self.pairs, self.prev_state, self.mul_prev,
                                                     self.mul_cur)
        x, kept = self.rt.ops.hashed_pair_embedding(ctx, self.weight, self.pairs, self.prev_state, self.mul_prev,
                                                    self.mul_cur, keep=True)
        ctx.aux["embedding_output"] = kept
        return x


@register_part("head", "lm_head")
class LMHead(Part):
    """``weight_name`` is the full checkpoint name of the [V, H] matrix: the head's own, or the
    embedding table's when the two are tied (the loader then shares one device tensor). ``logit_scale`` multiplies the
    logits; ``softcap`` c > 0 then bounds them, c tanh(logits / c) (one elementwise kernel behind the product)."""

    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, vocab_size: int, hidden_size: int, weight_name: Optional[str] = None,
                 bias: bool = False, logit_scale: float = 1.0, softcap: float = 0.0):
        super().__init__(prefix, rt)
        self.logit_scale, self.softcap = float(logit_scale), float(softcap)
        if self.softcap < 0:
            raise ValueError("lm_head: softcap must be >= 0")
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight_name = weight_name or "%s.weight" % prefix
        self.bias_name = "%s.bias" % prefix if bias else None
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        out = {self.weight_name: TensorDecl((self.vocab_size, self.hidden_size))}
        if self.bias_name:
            out[self.bias_name] = TensorDecl((self.vocab_size,))
        return out

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).contiguous()
        if self.bias_name:
            self.bias = fetch(self.bias_name).to(self.weight.dtype).contiguous()

    def forward(self, h: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """[R, H] -> float32 logits [R, V], written into ``out`` if one is given."""
        if out is not None:
            y = self.rt.ops.linear(h, self.weight, self.bias, out_dtype=torch.float32, out=out)
        else:
            y = self.rt.ops.linear(h, self.weight, self.bias, out_dtype=torch.float32)
        if self.logit_scale != 1.0 or self.softcap > 0.0:
            self.rt.ops.logit_cap(y, self.logit_scale, self.softcap)
        return y
