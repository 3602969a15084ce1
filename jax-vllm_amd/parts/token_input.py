"""A per-layer input that is looked up by the token itself (no reference counterpart).

Behind a layer's sublayers every token adds something of its own to the stream x:

    s = columns [offset, offset + dim) of row ``token`` of a table that all layers share
    y = W_proj ( act(W_gate x) * s )
    x <- x + norm(y)

The part computes y; the arrangement that holds it hands y on with this part's norm weight, so that the next
norm's kernel norms it, adds it to the float stream and norms the stream in one pass.  The table
``[vocab, table_width]`` belongs to the model: every layer's part declares it under the same checkpoint
name (``LayerSpec.shared``) and is handed the same buffer.  The token ids come with the step's context
(``StepContext.token_ids``); the activation runs in float.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import TensorSpec, register_part


class GatedTokenInput:
    replayable = True

    def __init__(self, hidden_size: int, vocab_size: int, dim: int, table_width: int, offset: int, eps: float,
                 activation: str = "gelu_tanh"):
        self.hidden_size, self.vocab_size, self.dim = int(hidden_size), int(vocab_size), int(dim)
        self.table_width, self.offset, self.eps = int(table_width), int(offset), float(eps)
        if activation not in K.PLAIN_ACTIVATIONS or activation is None:
            raise ValueError(f"no kernel for the activation {activation!r}")
        if self.dim < 1 or self.offset < 0 or self.offset + self.dim > self.table_width:
            raise ValueError(f"columns [{self.offset}, {self.offset + self.dim}) lie outside a table of width {self.table_width}")
        self.activation = activation
        self.table = self.w_gate = self.w_proj = self.norm_weight = None

    def tensors(self) -> dict:
        return {
            "table": TensorSpec((self.vocab_size, self.table_width)),
            "gate.weight": TensorSpec((self.dim, self.hidden_size)),
            "proj.weight": TensorSpec((self.hidden_size, self.dim)),
            "norm.weight": TensorSpec((self.hidden_size,), role="vector", init="norm"),
        }

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.table, self.w_gate, self.w_proj = tensors["table"], tensors["gate.weight"], tensors["proj.weight"]
        self.norm_weight = tensors["norm.weight"]

    def forward(self, x: torch.Tensor, ctx):
        """x: the stream in the activation type.  Returns y (rows, or a float stack of partial products)."""
        if ctx.token_ids is None:
            raise ValueError("a per-layer token input needs the step's token ids (StepContext.token_ids)")
        z = K.linear(x, self.w_gate)
        K.token_gate_mul(z, self.table, ctx.token_ids, self.offset, self.activation)
        return K.linear(z, self.w_proj, partial_ok=True)


register_part("token_input", "gated_token_input", GatedTokenInput)
