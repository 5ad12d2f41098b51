"""Token embedding and the language-model head.

Embedding: ``h0 = E[ids]`` (reference: src/forge_engine/qwen3.py:325), widened
to the float32 residual stream.  Head: ``logits = z @ W^T`` in float32, with W
the embedding matrix when tied (qwen3.py:336) or ``lm_head.weight`` otherwise;
only the rows that the step asks for are multiplied.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from ..cache.spec import CacheNeeds, CacheView, FixedState
from .base import BuildContext, Embedding, Head, ParamSpec, Residual


class TokenEmbedding(Embedding):
    def __init__(self, ctx: BuildContext, prefix: str, *, vocab_size: int, hidden_size: int,
                 leaf: str = "weight", scale: float = 1.0) -> None:
        """``scale``: a factor on every row as it enters the float32 stream."""
        super().__init__(ctx, prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.leaf = leaf        # the table's name behind the prefix ("": the prefix itself)
        self.scale = float(scale)
        self.weight: Tensor | None = None

    def param_specs(self):
        return {self.name(self.leaf): ParamSpec((self.vocab_size, self.hidden_size))}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name != self.name(self.leaf):
            raise KeyError(name)
        self.weight = tensor

    def forward(self, batch) -> Residual:
        h = torch.empty((batch.num_tokens, self.hidden_size), dtype=torch.float32, device=self.weight.device)
        ops.embed_rows(batch.token_ids, self.weight, h, self.scale)
        return Residual(h)

    def kernel_libraries(self):
        return {"rowwise"}


class TokenPairEmbedding(TokenEmbedding):
    """The token's row plus a row of a second table chosen by the token and the one before it:
    row ``(prev * mul_prev + cur * mul_cur) mod buckets``, and for a sequence's first token the
    table's last row (number ``buckets``).  The previous token is fixed-size state of the request
    (one integer a slot), so a request may be cut into steps anywhere."""

    PREVIOUS = "previous_token"

    def __init__(self, ctx: BuildContext, prefix: str, *, vocab_size: int, hidden_size: int, buckets: int,
                 mul_prev: int, mul_cur: int, leaf: str = "weight", pair_name: str = "pairs") -> None:
        """``pair_name``: the second table's full name in the checkpoint."""
        super().__init__(ctx, prefix, vocab_size=vocab_size, hidden_size=hidden_size, leaf=leaf)
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        self.pair_name = pair_name
        self.pair_weight: Tensor | None = None

    def param_specs(self):
        return dict(super().param_specs(), **{self.pair_name: ParamSpec((self.buckets + 1, self.hidden_size))})

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name == self.pair_name:
            self.pair_weight = tensor
        else:
            super().set_param(name, tensor)

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(state={self.PREVIOUS: FixedState((1,), torch.int32)})

    def forward(self, batch, cache: CacheView | None = None) -> Residual:
        h = torch.empty((batch.num_tokens, self.hidden_size), dtype=torch.float32, device=self.weight.device)
        ops.embed_token_pairs(batch.token_ids, self.weight, self.pair_weight, batch.positions, batch.token_seq, batch.cu_q,
                              batch.state_slots, cache.states[self.PREVIOUS], h, num_seqs=batch.num_seqs,
                              buckets=self.buckets, mul_prev=self.mul_prev, mul_cur=self.mul_cur)
        return Residual(h)

    def kernel_libraries(self):
        return {"rowwise", "hyper"}


class LMHead(Head):
    def __init__(self, ctx: BuildContext, prefix: str, *, vocab_size: int, hidden_size: int,
                 tied: bool = False, leaf: str = "weight", scale: float = 1.0) -> None:
        """``scale``: a factor on the logits."""
        super().__init__(ctx, prefix)
        self.scale = float(scale)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied
        self.leaf = leaf
        self.weight: Tensor | None = None
        self._embedding: TokenEmbedding | None = None

    def tie(self, embedding: TokenEmbedding) -> None:
        self._embedding = embedding

    def param_specs(self):
        if self.tied:
            return {}
        return {self.name(self.leaf): ParamSpec((self.vocab_size, self.hidden_size))}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if self.tied or name != self.name(self.leaf):
            raise KeyError(name)
        self.weight = tensor

    def matrix(self) -> Tensor:
        return self._embedding.weight if self.tied else self.weight

    def forward(self, z: Tensor) -> Tensor:
        # float32 accumulation and float32 logits in both modes (no rounding of the logits)
        logits = ops.linear(z, self.matrix(), out_dtype=torch.float32)
        return logits if self.scale == 1.0 else ops.scale_rows(logits, self.scale)

    def kernel_libraries(self):
        return {"gemm_f32", "gemm_skinny"} | ({"hyper"} if self.scale != 1.0 else set())


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("embedding", "token_pair_embedding", TokenPairEmbedding)
register_part("head", "lm_head", LMHead)
