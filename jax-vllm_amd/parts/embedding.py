"""Token embedding and output head.  Reference: ``jllm/model/common.py:35-41`` (row gather,
``x @ W.T`` without bias) and ``jllm/model/weights.py:143-146`` (a tied head is the
embedding table itself, one buffer)."""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import TensorSpec, register_part


class TokenEmbedding:
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0):
        """``scale``: a constant on every row, multiplied in float."""
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.scale = float(scale)
        self.weight = None

    def tensors(self) -> dict:
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.weight = tensors["weight"]

    def forward(self, ids: torch.Tensor, ctx=None) -> torch.Tensor:
        """Float residual stream [tokens, hidden] of the rows ``ids`` (int32; an id outside the table
        gives a row of NaN).  ``ctx`` is the step's ``StepContext`` (positions, token -> request, ...);
        this embedding needs none of it."""
        h = torch.empty((ids.numel(), self.hidden_size), dtype=torch.float32, device=ids.device)
        if self.scale != 1.0:
            if ctx is None or ctx.prev_tokens is None:
                raise ValueError("a scaled embedding runs through the pair kernel, which reads StepContext.prev_tokens")
            K.embedding_pair(h, self.weight, None, ids, ctx.prev_tokens, 1, 0, 0, scale=self.scale)
        else:
            K.embedding(h, self.weight, ids)
        return h


class TokenPairEmbedding(TokenEmbedding):
    """The token's row plus a row of a second table chosen by the pair (previous token, token):
    row ``(previous * mul_prev + token * mul_cur) mod buckets``; a sequence's first token takes the table's
    spare last row (number ``buckets``).  The previous token of every token of the step comes with the step's
    context (``StepContext.prev_tokens``, -1 for a first token): for the first token of a portion it is the last
    token the cache manager holds for the request.  ``scale``: a constant on the token's own row (not on the pair's).
    The sum is float."""

    def __init__(self, vocab_size: int, hidden_size: int, buckets: int, mul_prev: int, mul_cur: int,
                 pair_name: str = "pair.weight", scale: float = 1.0):
        super().__init__(vocab_size, hidden_size, scale)
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        if self.buckets < 1 or self.mul_prev < 0 or self.mul_cur < 0:
            raise ValueError("buckets must be positive and the multipliers non-negative")
        self.pair_name = pair_name
        self.pair = None

    def tensors(self) -> dict:
        t = super().tensors()
        t[self.pair_name] = TensorSpec((self.buckets + 1, self.hidden_size))
        return t

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        super().bind(tensors, dtype)
        self.pair = tensors[self.pair_name]

    def forward(self, ids: torch.Tensor, ctx=None) -> torch.Tensor:
        if ctx is None or ctx.prev_tokens is None:
            raise ValueError("this embedding needs every token's previous token (StepContext.prev_tokens)")
        h = torch.empty((ids.numel(), self.hidden_size), dtype=torch.float32, device=ids.device)
        K.embedding_pair(h, self.weight, self.pair, ids, ctx.prev_tokens, self.buckets, self.mul_prev, self.mul_cur,
                         scale=self.scale)
        return h


class LinearHead:
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int, softcap: float | None = None):
        """``softcap`` c: logits <- c tanh(logits / c)."""
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.softcap = float(softcap) if softcap else None
        self.weight = None

    def tensors(self) -> dict:
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Float logits [rows, vocab]."""
        z = K.linear(x, self.weight, out_dtype=torch.float32)
        return K.softcap(z, self.softcap) if self.softcap else z


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("embedding", "token_pair_embedding", TokenPairEmbedding)
register_part("head", "linear_head", LinearHead)
