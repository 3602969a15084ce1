"""Mixers that keep a float matrix state per request and head instead of a cache of keys (no reference
counterpart).  All three run ONE recurrence, ``K.recurrence_steps``,

    S <- g S;   u = w (v - [delta] S^T k);   S <- S + k u^T;   o = S^T q (+ skip v)

and differ in what q, k, v, the decay g and the write strength w are made of:

* ``retention``:   q, k rotated by position, k / sqrt(dim); g a constant per head, w = 1; every head's o divided by its
                   own root mean square (no weight), times silu(gate).
* ``state_space``: (Mamba-2) one input product cut into [z | x | B | C | dt]; x, B, C through a short causal
                   convolution with bias and silu; dt = softplus(dt + bias), g = exp(-exp(A) dt), w = dt; k = B and q = C
                   are shared by a group of heads, v = x; skip D; o * silu(z) normed in equal groups with a weight.
* ``gated_delta``: q, k, v through short convolutions and silu; q, k unit vectors per head, q / sqrt(dim); g as above
                   from a projection of its own, w = sigmoid(another projection); delta = 1; every head's o normed with a
                   weight shared by the heads, times silu(gate).

A fourth mixer, ``time_mix`` (below), has a recurrence of its own, ``K.wkv_steps``: a decay per key channel instead of
one per head, the output read from the state BEFORE the token's update, and a bonus on the token's own key.

Everything that enters the recurrence is float (the products and the convolutions' results are in the activation
type).  The state, and the last taps - 1 inputs of every convolution, live in the request's state slot between steps.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..ops import kernels as K
from .spec import LayerMemory, PartSpec, StateSpec, StepContext, TensorSpec, build_part, is_replayable, register_part


class Retention:
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_dim: int, decay: Sequence[float], norm_eps: float,
                 position: Optional[PartSpec] = None, out_scale: float = 1.0):
        self.hidden_size, self.heads, self.dim, self.vdim = int(hidden_size), int(num_heads), int(head_dim), int(v_dim)
        self.decay_values = [float(d) for d in decay]
        if len(self.decay_values) != self.heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.heads} heads")
        self.eps, self.out_scale = float(norm_eps), float(out_scale)
        self.position = build_part("position", position) if position is not None else None
        rotation = self.position.as_rotation() if self.position is not None else None
        if rotation is not None and rotation[1]:
            raise ValueError("the recurrence's input kernel rotates half-split pairs (i, i + dims/2) only")
        self.rot_dims = int(rotation[0]) if rotation is not None else 0

    @property
    def replayable(self) -> bool:
        return self.position is None or is_replayable(self.position)

    def tensors(self) -> dict:
        H, hid = self.heads, self.hidden_size
        return {
            "q_proj.weight": TensorSpec((H * self.dim, hid)),
            "k_proj.weight": TensorSpec((H * self.dim, hid)),
            "v_proj.weight": TensorSpec((H * self.vdim, hid)),
            "gate.weight": TensorSpec((H * self.vdim, hid)),
            "o_proj.weight": TensorSpec((hid, H * self.vdim)),
        }

    def cache_spec(self):
        return None

    def state_spec(self):
        return StateSpec((self.heads, self.dim, self.vdim), "float32", "S")

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        self.w_in = torch.cat([tensors[k + ".weight"] for k in ("q_proj", "k_proj", "v_proj", "gate")], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=self.w_o.device)
        if self.position is not None:
            self.position.bind({}, dtype, self.w_o.device)

    def forward(self, x, ctx: StepContext, mem: LayerMemory):
        H, d, dv = self.heads, self.dim, self.vdim
        proj = K.linear(x, self.w_in)
        cos_sin = self.position.rotation_table(ctx) if self.rot_dims else None
        qkv = K.qkv_to_f32(proj, H, d, dv, self.rot_dims, cos_sin, k_scale=d ** -0.5)
        q, k, v = qkv[:, :H * d], qkv[:, H * d:2 * H * d], qkv[:, 2 * H * d:]
        o = K.recurrence_steps(q, k, v, self.decay, mem.states["S"], ctx.slot_ids, ctx.cu_seqlens, H, H, d, dv,
                               chunk_plan=K.step_chunk_plan(ctx, d))
        y = K.group_gated_norm(o, proj[:, 2 * H * d + H * dv:], None, dv, self.eps, "silu", out_scale=self.out_scale)
        return K.linear(y, self.w_o, partial_ok=True)


class StateSpaceMixer:
    replayable = True     # slots, request borders and tokens come from the device; the kernel choice does not depend on values

    def __init__(self, hidden_size: int, num_heads: int, v_dim: int, state_size: int, groups: int, conv_taps: int,
                 norm_groups: int, norm_eps: float, out_scale: float = 1.0):
        self.hidden_size, self.heads, self.vdim, self.n = int(hidden_size), int(num_heads), int(v_dim), int(state_size)
        self.groups, self.taps, self.norm_groups = int(groups), int(conv_taps), int(norm_groups)
        self.eps, self.out_scale = float(norm_eps), float(out_scale)
        self.inner = self.heads * self.vdim
        if self.heads % self.groups:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.groups} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"an inner size of {self.inner} does not split into {self.norm_groups} equal parts")
        self.channels = self.inner + 2 * self.groups * self.n

    def tensors(self) -> dict:
        return {
            "in_proj.weight": TensorSpec((2 * self.inner + 2 * self.groups * self.n + self.heads, self.hidden_size)),
            "conv.weight": TensorSpec((self.channels, self.taps), role="vector"),
            "conv.bias": TensorSpec((self.channels,), role="vector"),
            "dt_bias": TensorSpec((self.heads,), role="vector"),
            "A_log": TensorSpec((self.heads,), role="vector", init="log_rate"),
            "D": TensorSpec((self.heads,), role="vector", init="norm"),
            "norm.weight": TensorSpec((self.inner,), role="vector", init="norm"),
            "o_proj.weight": TensorSpec((self.hidden_size, self.inner)),
        }

    def cache_spec(self):
        return None

    def state_spec(self):
        return (StateSpec((self.heads, self.n, self.vdim), "float32", "S"),
                StateSpec((self.taps - 1, self.channels), "float32", "conv"))

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        self.w_in, self.w_o = tensors["in_proj.weight"], tensors["o_proj.weight"]
        self.conv_w, self.conv_b = tensors["conv.weight"].contiguous(), tensors["conv.bias"]
        self.dt_bias, self.a_log, self.skip = tensors["dt_bias"], tensors["A_log"], tensors["D"]
        self.norm_weight = tensors["norm.weight"]

    def forward(self, x, ctx: StepContext, mem: LayerMemory):
        H, dv, N, G, inner = self.heads, self.vdim, self.n, self.groups, self.inner
        proj = K.linear(x, self.w_in)                       # [z | x | B | C | dt]
        xbc = K.short_conv(proj, inner, self.channels, self.conv_w, self.conv_b, mem.states["conv"], ctx.slot_ids,
                           ctx.cu_seqlens, ctx.max_q_len)
        g, dt = K.recurrence_gates(proj, inner + self.channels, self.dt_bias, self.a_log, H)
        v, b, c = xbc[:, :inner], xbc[:, inner:inner + G * N], xbc[:, inner + G * N:]
        o = K.recurrence_steps(c, b, v, g, mem.states["S"], ctx.slot_ids, ctx.cu_seqlens, H, G, N, dv, write=dt, skip=self.skip,
                               chunk_plan=K.step_chunk_plan(ctx, N))
        y = K.group_gated_norm(o, proj[:, :inner], self.norm_weight, inner // self.norm_groups, self.eps, "silu",
                               gate_first=True, out_scale=self.out_scale)
        return K.linear(y, self.w_o, partial_ok=True)


class GatedDeltaMixer:
    replayable = True

    def __init__(self, hidden_size: int, num_heads: int, num_qk_heads: int, head_dim: int, v_dim: int, conv_taps: int,
                 norm_eps: float, unit_eps: float = 1e-6, out_scale: float = 1.0):
        self.hidden_size, self.heads, self.qk_heads = int(hidden_size), int(num_heads), int(num_qk_heads)
        self.dim, self.vdim, self.taps = int(head_dim), int(v_dim), int(conv_taps)
        self.eps, self.unit_eps, self.out_scale = float(norm_eps), float(unit_eps), float(out_scale)
        if self.heads % self.qk_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.qk_heads} q/k heads")
        self.qk, self.inner = self.qk_heads * self.dim, self.heads * self.vdim
        self.channels = 2 * self.qk + self.inner

    def tensors(self) -> dict:
        hid = self.hidden_size
        return {
            "q_proj.weight": TensorSpec((self.qk, hid)),
            "k_proj.weight": TensorSpec((self.qk, hid)),
            "v_proj.weight": TensorSpec((self.inner, hid)),
            "q_conv.weight": TensorSpec((self.qk, self.taps), role="vector"),
            "k_conv.weight": TensorSpec((self.qk, self.taps), role="vector"),
            "v_conv.weight": TensorSpec((self.inner, self.taps), role="vector"),
            "beta_proj.weight": TensorSpec((self.heads, hid)),
            "decay_proj.weight": TensorSpec((self.heads, hid)),
            "dt_bias": TensorSpec((self.heads,), role="vector"),
            "A_log": TensorSpec((self.heads,), role="vector", init="log_rate"),
            "gate.weight": TensorSpec((self.inner, hid)),
            "norm.weight": TensorSpec((self.vdim,), role="vector", init="norm"),
            "o_proj.weight": TensorSpec((hid, self.inner)),
        }

    def cache_spec(self):
        return None

    def state_spec(self):
        return (StateSpec((self.heads, self.dim, self.vdim), "float32", "S"),
                StateSpec((self.taps - 1, self.channels), "float32", "conv"))

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        # one product for everything that reads the input: [q | k | v | gate | decay | beta]
        self.w_in = torch.cat([tensors[k + ".weight"] for k in ("q_proj", "k_proj", "v_proj", "gate", "decay_proj", "beta_proj")],
                              dim=0).contiguous()
        self.conv_w = torch.cat([tensors[k + "_conv.weight"] for k in ("q", "k", "v")], dim=0).contiguous()
        self.dt_bias, self.a_log, self.norm_weight = tensors["dt_bias"], tensors["A_log"], tensors["norm.weight"]
        self.w_o = tensors["o_proj.weight"]

    def forward(self, x, ctx: StepContext, mem: LayerMemory):
        H, d, dv, qk, inner = self.heads, self.dim, self.vdim, self.qk, self.inner
        proj = K.linear(x, self.w_in)
        qkv = K.short_conv(proj, 0, self.channels, self.conv_w, None, mem.states["conv"], ctx.slot_ids, ctx.cu_seqlens,
                           ctx.max_q_len)
        gate_at = self.channels
        g, beta = K.recurrence_gates(proj, gate_at + inner, self.dt_bias, self.a_log, H, beta_off=gate_at + inner + H)
        q, k, v = qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:]
        K.head_unit_norm(qkv, 2 * self.qk_heads, d, self.unit_eps, 1.0, first_heads=self.qk_heads, first_scale=d ** -0.5)
        o = K.recurrence_steps(q, k, v, g, mem.states["S"], ctx.slot_ids, ctx.cu_seqlens, H, self.qk_heads, d, dv,
                               write=beta, delta=True, chunk_plan=K.step_chunk_plan(ctx, d, delta=True))
        y = K.group_gated_norm(o, proj[:, gate_at:gate_at + inner], self.norm_weight, dv, self.eps, "silu",
                               out_scale=self.out_scale)
        return K.linear(y, self.w_o, partial_ok=True)


class TimeMix:
    """Time mixing with token shift, a data-dependent decay per key channel and a bonus for the current token.  With h_t
    the mixer's input and h_(t-1) the row before it in the request (zeros before the first token), each of r, k, v, g, w
    reads a blend of its own, b_s = h_t + (h_(t-1) - h_t) * mu_s:

        r, k, v = W_r b_r, W_k b_k, W_v b_v  [heads, dim];   gate = silu(W_g b_g)
        decay   = exp(-exp(W_w2 tanh(W_w1 b_w) + w0))         per head and key channel, float
        o_t     = S^T r_t + (sum_d r_t[d] u[d] k_t[d]) v_t;    S <- diag(decay_t) S + k_t v_t^T      per head, S [dim, dim] float
        out     = W_o ( concat_h( o_t / rms(o_t) ) * norm * gate )

    The state S and the last input row h live in the request's state slot between steps (``S`` and ``shift``)."""

    replayable = True     # slots, request borders and tokens come from the device; the kernel choice does not depend on values

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, norm_eps: float, decay_rank: Optional[int] = None):
        """``decay_rank`` None: the inner size of the decay's two products is whatever the checkpoint's tensors have."""
        self.hidden_size, self.heads, self.dim = int(hidden_size), int(num_heads), int(head_dim)
        self.decay_rank, self.eps = int(decay_rank) if decay_rank else None, float(norm_eps)
        if self.dim > K.WKV_MAX_DIM:
            raise ValueError(f"the recurrence keeps heads of at most {K.WKV_MAX_DIM} channels, not {self.dim}")
        self.inner = self.heads * self.dim

    def tensors(self) -> dict:
        hid, inner = self.hidden_size, self.inner
        t = {f"mu.{s}": TensorSpec((hid,), role="vector", init="fraction") for s in self.MIXES}
        t.update({
            "r_proj.weight": TensorSpec((inner, hid)),
            "k_proj.weight": TensorSpec((inner, hid)),
            "v_proj.weight": TensorSpec((inner, hid)),
            "gate.weight": TensorSpec((inner, hid)),
            "decay_down.weight": TensorSpec((self.decay_rank, hid)),
            "decay_up.weight": TensorSpec((inner, self.decay_rank)),
            "decay_base": TensorSpec((inner,), role="vector", init="log_rate"),
            "bonus": TensorSpec((self.heads, self.dim), role="vector", init="norm"),
            "norm.weight": TensorSpec((inner,), role="vector", init="norm"),
            "o_proj.weight": TensorSpec((hid, inner)),
        })
        return t

    def cache_spec(self):
        return None

    def state_spec(self):
        return (StateSpec((self.heads, self.dim, self.dim), "float32", "S"),
                StateSpec((self.hidden_size,), "float32", "shift"))

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        self.mu = torch.stack([tensors[f"mu.{s}"] for s in self.MIXES]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (tensors[k + ".weight"] for k in ("r_proj", "k_proj", "v_proj", "gate"))
        self.w_decay_down, self.w_decay_up = tensors["decay_down.weight"], tensors["decay_up.weight"]
        self.decay_base = tensors["decay_base"].contiguous()
        self.bonus = tensors["bonus"].reshape(-1).contiguous()
        self.norm_weight, self.w_o = tensors["norm.weight"], tensors["o_proj.weight"]

    def forward(self, x, ctx: StepContext, mem: LayerMemory):
        H, d = self.heads, self.dim
        b = K.token_shift_mix(x, self.mu, mem.states["shift"], ctx.slot_ids, ctx.cu_seqlens, ctx.token_req)
        r, k, v, gate = (K.linear(b[i], w) for i, w in enumerate((self.w_r, self.w_k, self.w_v, self.w_g)))
        low = K.linear(b[4], self.w_decay_down)
        K.bias_act(low, None, "tanh")
        rate = K.linear(low, self.w_decay_up)
        o = K.wkv_steps(r, k, v, rate, self.decay_base, self.bonus, mem.states["S"], ctx.slot_ids, ctx.cu_seqlens, H, d, d,
                        chunk_plan=K.wkv_chunk_plan(ctx, d))
        y = K.group_gated_norm(o, gate, self.norm_weight, d, self.eps, "silu")
        return K.linear(y, self.w_o, partial_ok=True)


class ParallelMixer:
    """Two mixers side by side on the same input: ``left_scale * left(x) + right_scale * right(x)``.  Either may keep
    pages, either may keep state (their state tensors are declared under ``left.`` and ``right.``); their results
    go on as a float stack of two weighed shares that the next norm adds."""

    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0):
        self.sides = (("left.", build_part("mixer", left), float(left_scale)),
                      ("right.", build_part("mixer", right), float(right_scale)))
        if sum(part.cache_spec() is not None for _, part, _ in self.sides) > 1:
            raise ValueError("two mixers side by side that both keep pages: a layer has one paged cache")

    @property
    def replayable(self) -> bool:
        return all(is_replayable(part) for _, part, _ in self.sides)

    def tensors(self) -> dict:
        return {prefix + name: ts for prefix, part, _ in self.sides for name, ts in part.tensors().items()}

    def cache_spec(self):
        return next((part.cache_spec() for _, part, _ in self.sides if part.cache_spec() is not None), None)

    def state_spec(self):
        from .spec import state_specs_of

        specs = tuple(StateSpec(st.shape, st.dtype, prefix + st.name)
                      for prefix, part, _ in self.sides for st in state_specs_of(part.state_spec()))
        return specs or None

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        for prefix, part, _ in self.sides:
            part.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}, dtype)

    def forward(self, x, ctx: StepContext, mem: LayerMemory):
        out = torch.empty((len(self.sides), x.shape[0], x.shape[1]), dtype=torch.float32, device=x.device)
        for i, (prefix, part, scale) in enumerate(self.sides):
            K.scaled_sum(out[i], part.forward(x, ctx, mem.below(prefix)), scale)
        return out


register_part("mixer", "retention", Retention)
register_part("mixer", "state_space", StateSpaceMixer)
register_part("mixer", "gated_delta", GatedDeltaMixer)
register_part("mixer", "time_mix", TimeMix)
register_part("mixer", "parallel", ParallelMixer)
