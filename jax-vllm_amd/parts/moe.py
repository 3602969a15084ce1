"""Routed experts: a feed-forward of many small gated feed-forwards, of which each token uses a few
(no reference counterpart).

    z = W_router x (+ b)  (float);   the ``top`` experts with the largest z are chosen;
    s = sigmoid(z), or (``score`` "softmax_chosen") the softmax over the chosen z alone, or (``score``
    "sigmoid_normed") the experts with the largest sigmoid(z) + correction are chosen and
    s = sigmoid(z) / (sum of the chosen sigmoids + 1e-20) * ``weight_scale``
    out = sum over the chosen e of  expert_e(s_e * x)   [+ shared(x)  or  + sigmoid(w_sg . x) shared(x)]
    expert(u) = W_down ( act(W_gate u) * (W_up u) )

The score multiplies the expert's INPUT (``weight_on_input``; with False it multiplies the output).  Since
the products are linear, s (W u) is computed instead of W (s u): in float, after the product.  Routing,
the grouping of rows by expert and the two grouped products all run on the device (``ops.kernels.moe_*``).
The result is handed on as (rows of the shared expert or None, float stack [top, tokens, hidden] of the
chosen experts' outputs); the next norm adds them in that order.  A shared expert under a gate of the token's own
(``shared_gate``) joins the float stack as one more share.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .spec import PartSpec, TensorSpec, build_part, is_replayable, register_part


class RoutedExperts:
    def __init__(self, hidden_size: int, num_experts: int, top: int, expert_size: int, activation: str = "silu",
                 weight_on_input: bool = True, shared: Optional[PartSpec] = None,
                 expert_names=("gate", "up", "down"), router_bias: bool = False, score: str = "sigmoid",
                 choice_correction: bool = False, weight_scale: float = 1.0, shared_gate: bool = False):
        if activation not in K.GATE_ACTIVATIONS:
            raise ValueError(f"the expert kernels have {sorted(K.GATE_ACTIVATIONS)}, not {activation!r}")
        self.hidden_size, self.experts, self.top, self.ff = int(hidden_size), int(num_experts), int(top), int(expert_size)
        if not 0 < self.top <= self.experts:
            raise ValueError(f"top = {self.top} of {self.experts} experts")
        if score not in K.ROUTER_SCORES:
            raise ValueError(f"the router kernels have the scores {sorted(K.ROUTER_SCORES)}, not {score!r}")
        self.activation, self.weight_on_input = activation, bool(weight_on_input)
        self.router_bias, self.score = bool(router_bias), score
        self.choice_correction, self.weight_scale = bool(choice_correction), float(weight_scale)
        if (self.choice_correction or self.weight_scale != 1.0) and score != "sigmoid_normed":
            raise ValueError("a correction of the choice and a constant on the weights belong to the score 'sigmoid_normed'")
        self.shared_gate = bool(shared_gate)
        if self.shared_gate and shared is None:
            raise ValueError("a gate on the shared expert without a shared expert")
        self.b_router = self.correction = self.w_shared_gate = None
        self.names = tuple(expert_names)
        self.shared = build_part("feed_forward", shared) if shared is not None else None
        if self.shared is not None and hasattr(self.shared, "partial_out"):
            self.shared.partial_out = False     # its rows are added beside the experts' float stack

    @property
    def replayable(self) -> bool:
        return self.shared is None or is_replayable(self.shared)

    def tensors(self) -> dict:
        g, u, d = self.names
        t = {"router.weight": TensorSpec((self.experts, self.hidden_size))}
        if self.router_bias:
            t["router.bias"] = TensorSpec((self.experts,), role="vector")
        for e in range(self.experts):
            t[f"experts.{e}.{g}.weight"] = TensorSpec((self.ff, self.hidden_size))
            t[f"experts.{e}.{u}.weight"] = TensorSpec((self.ff, self.hidden_size))
            t[f"experts.{e}.{d}.weight"] = TensorSpec((self.hidden_size, self.ff))
        if self.choice_correction:
            t["router.correction"] = TensorSpec((self.experts,), role="vector", init="small")
        if self.shared is not None:
            for k, v in self.shared.tensors().items():
                t["shared." + k] = v
        if self.shared_gate:
            t["shared_gate.weight"] = TensorSpec((1, self.hidden_size))
        return t

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        g, u, d = self.names
        self.w_router = tensors["router.weight"]
        if self.router_bias:
            self.b_router = tensors["router.bias"].contiguous()
        self.w_gate = torch.stack([tensors[f"experts.{e}.{g}.weight"] for e in range(self.experts)]).contiguous()
        self.w_up = torch.stack([tensors[f"experts.{e}.{u}.weight"] for e in range(self.experts)]).contiguous()
        self.w_down = torch.stack([tensors[f"experts.{e}.{d}.weight"] for e in range(self.experts)]).contiguous()
        if self.choice_correction:
            self.correction = tensors["router.correction"].contiguous()
        if self.shared is not None:
            self.shared.bind({k[len("shared."):]: v for k, v in tensors.items() if k.startswith("shared.")}, dtype)
        if self.shared_gate:
            w = tensors["shared_gate.weight"]
            self.w_shared_gate = torch.cat([w, w.new_zeros((7, w.shape[1]))]).contiguous()   # rows of 16 bytes and more

    def forward(self, x, ctx=None):
        n = x.shape[0]
        plan = K.moe_route(None, self.top, x=x, w_router=self.w_router, bias=self.b_router, score=self.score,
                           tile_rows=K.moe_tile_rows_for(x.dtype, self.hidden_size, self.ff, n * self.top, self.experts),
                           correction=self.correction, weight_scale=self.weight_scale)
        shares = self.top + (1 if self.shared_gate else 0)
        out = torch.empty((shares, n, self.hidden_size), dtype=torch.float32, device=x.device)
        K.moe_experts(x, plan, self.w_gate, self.w_up, self.w_down, self.activation, out[:self.top], self.weight_on_input)
        rows = self.shared.forward(x, ctx) if self.shared is not None else None
        if self.shared_gate:
            K.row_gate(out[self.top], rows, K.linear(x, self.w_shared_gate)[:, :1])
            rows = None
        return rows, out


register_part("feed_forward", "routed_experts", RoutedExperts)
