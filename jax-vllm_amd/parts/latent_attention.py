"""Attention through a low-rank latent, over a paged cache of that latent (no reference counterpart).

A token's keys and values of ALL heads are functions of one vector per token:

    c      = norm(W_dkv h)[:rank]                       the latent, cached
    k_rot  = rotate(W_dkv h [rank:])                    one rotated key part shared by the heads, cached
    k[h]   = [W_uk[h] c | k_rot],   v[h] = W_uv[h] c
    q[h]   = W_uq[h] norm(W_dq h) = [q_plain | q_rot], q_rot rotated
    score  = (q_plain . W_uk[h] c + q_rot . k_rot) * scale,   causal, optionally a sliding window
    out    = W_o ( concat_h(softmax . v[h]) * sigmoid(W_g h) )      (the gate is an option)

Since q_plain . (W_uk[h] c) = (W_uk[h]^T q_plain) . c and sum_j p_j W_uv[h] c_j = W_uv[h] sum_j p_j c_j,
the cached vector e = [c | k_rot] serves as key AND value of one shared kv head of size rank + rot: the
paged attention kernels of grouped-query attention run unchanged (one kv head, ``heads`` q heads), on a
query [W_uk[h]^T q_plain | q_rot], and W_uv[h] is applied to the first ``rank`` elements of their result.
The same arithmetic serves prompts and decoded tokens, so logits do not depend on how a prompt is cut.
The cache keeps e in the two layouts those kernels read (``parts.spec.kv_cache_spec``).

Options: ``q_rank`` 0: the queries are projected directly, q = W_q h (no query latent, no query norm);
the rotation may pair (i, i + dims/2) or (2i, 2i + 1), as its position part says; ``sinks``: a learned number
per head whose exponential joins the softmax denominator (no key, no value, not scaled); ``output_gate``
"head": one gate per head, sigmoid(W_g h)_h with W_g [heads, hidden], instead of one per output element;
``own_cache`` False: the layer has no W_dkv and reads the cached vectors e of an earlier layer (the schedule's
``cache_of``), with its own W_uk, W_uv, queries and everything else.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .spec import LayerMemory, PagedCacheSpec, PartSpec, StepContext, TensorSpec, build_part, is_replayable, kv_cache_spec, register_part


class LatentAttention:
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, v_dim: int, q_rank: int,
                 kv_rank: int, scale: float, norm_eps: float, position: Optional[PartSpec] = None,
                 window: Optional[int] = None, output_gate="element", sinks: bool = False, own_cache: bool = True):
        self.hidden_size, self.heads = int(hidden_size), int(num_heads)
        self.dim, self.rot, self.vdim = int(head_dim), int(rot_dim), int(v_dim)
        self.q_rank, self.rank = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(norm_eps)
        self.window = int(window) if window else None
        if output_gate is True:
            output_gate = "element"
        if output_gate not in (None, False, "element", "head"):
            raise ValueError(f"output_gate is None, 'element' or 'head', not {output_gate!r}")
        self.output_gate = output_gate or None
        self.has_sinks, self.own_cache = bool(sinks), bool(own_cache)
        if self.q_rank < 0:
            raise ValueError("q_rank is the size of the query latent, or 0 for queries projected directly")
        self.position = build_part("position", position) if position is not None and self.rot else None
        rotation = self.position.as_rotation() if self.position is not None else None
        self.rot_dims = int(rotation[0]) if rotation is not None else 0
        self.interleaved = bool(rotation[1]) if rotation is not None else False
        if self.rot_dims > self.rot:
            raise ValueError(f"{self.rot_dims} rotated dimensions do not fit a key part of {self.rot}")
        # what the paged attention kernels see: one kv head of the cached vector's size
        self.nq, self.nkv, self.d = self.heads, 1, self.rank + self.rot
        self.q_row_stride = self.heads * self.d

    @property
    def replayable(self) -> bool:
        return self.position is None or is_replayable(self.position)

    def tensors(self) -> dict:
        H, hid = self.heads, self.hidden_size
        t = {
            "k_up.weight": TensorSpec((H * self.dim, self.rank)),
            "v_up.weight": TensorSpec((H * self.vdim, self.rank)),
            "o_proj.weight": TensorSpec((hid, H * self.vdim)),
        }
        if self.q_rank:
            t["q_down.weight"] = TensorSpec((self.q_rank, hid))
            t["q_norm.weight"] = TensorSpec((self.q_rank,), role="vector", init="norm")
            t["q_up.weight"] = TensorSpec((H * (self.dim + self.rot), self.q_rank))
        else:
            t["q_proj.weight"] = TensorSpec((H * (self.dim + self.rot), hid))
        if self.own_cache:
            t["kv_down.weight"] = TensorSpec((self.rank + self.rot, hid))
            t["kv_norm.weight"] = TensorSpec((self.rank,), role="vector", init="norm")
        if self.output_gate:
            t["gate.weight"] = TensorSpec((H if self.output_gate == "head" else H * self.vdim, hid))
        if self.has_sinks:
            t["sinks"] = TensorSpec((H,), role="vector", init="small")
        return t

    def cache_spec(self) -> Optional[PagedCacheSpec]:
        return kv_cache_spec(1, self.d, self.window)

    def state_spec(self):
        return None

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        H = self.heads
        # one product for everything that reads the input: [q latent, or q itself | kv latent, key part | gate]
        down = [tensors["q_down.weight"] if self.q_rank else tensors["q_proj.weight"]]
        self.kv_at = down[0].shape[0]
        self.gate_at = self.kv_at
        if self.own_cache:
            down.append(tensors["kv_down.weight"])
            self.gate_at += self.rank + self.rot
        if self.output_gate:
            down.append(tensors["gate.weight"])
        self.gate_width = H if self.output_gate == "head" else H * self.vdim
        rows = sum(d.shape[0] for d in down)
        if rows % 8:      # rows of the product stay 16-byte aligned for the kernels that read heads out of them
            down.append(down[0].new_zeros((8 - rows % 8, self.hidden_size)))
        self.w_down = torch.cat(down, dim=0).contiguous()
        self.q_norm = tensors["q_norm.weight"] if self.q_rank else None
        self.kv_norm = tensors["kv_norm.weight"] if self.own_cache else None
        self.w_q_up = tensors["q_up.weight"] if self.q_rank else None
        self.sinks = tensors["sinks"].contiguous() if self.has_sinks else None
        self.w_k_up_t = tensors["k_up.weight"].view(H, self.dim, self.rank).transpose(1, 2).contiguous()   # [H, rank, dim]
        self.w_v_up = tensors["v_up.weight"].view(H, self.vdim, self.rank).contiguous()
        self.w_o = tensors["o_proj.weight"]
        if self.position is not None:
            self.position.bind({}, dtype, self.w_o.device)

    def forward(self, x, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        n, H, E = x.shape[0], self.heads, self.d
        cos_sin = self.position.rotation_table(ctx) if self.rot_dims else None
        proj = K.linear(x, self.w_down)
        writes = mem.writes
        if writes != self.own_cache:
            raise ValueError("a latent attention layer writes the cache it declares, or reads another layer's and has no W_dkv")
        cq = None
        if self.own_cache:
            cq = K.latent_prepare(proj, self.q_rank, self.rank, self.rot, self.rot_dims, self.q_norm, self.kv_norm, self.eps,
                                  cos_sin, ctx.slot_mappings[mem.group], mem.pages["k"], mem.pages["v"], ctx.page_size,
                                  kv_off=self.kv_at, interleaved=self.interleaved)
        elif self.q_rank:
            cq = K.rmsnorm(proj[:, :self.q_rank].contiguous(), self.q_norm, self.eps)
        q = K.linear(cq, self.w_q_up) if self.q_rank else proj       # proj's rows begin with the queries
        qe = torch.empty((n, H * E), dtype=x.dtype, device=x.device)
        K.head_linear(qe, E, q, self.dim + self.rot, self.w_k_up_t)             # W_uk[h]^T q_plain
        if self.rot:
            K.latent_query_rope(q, qe, H, self.dim, self.rot, self.rot_dims, self.rank, cos_sin, self.interleaved)
        att = torch.empty((n, H * E), dtype=x.dtype, device=x.device)
        from . import attention_backend

        attention_backend.run(self, att, qe, ctx, mem)
        o = torch.empty((n, H * self.vdim), dtype=x.dtype, device=x.device)
        gate = proj[:, self.gate_at:self.gate_at + self.gate_width] if self.output_gate else None
        K.head_linear(o, self.vdim, att, E, self.w_v_up, gate=gate)
        return K.linear(o, self.w_o, partial_ok=True)


register_part("mixer", "latent_attention", LatentAttention)
