"""Pre-norm residual arrangement of one layer.  Reference: ``jllm/model/common.py:140-147``:

    h = h + mixer(norm_1(h));   h = h + feed_forward(norm_2(h))

The residual stream ``h`` is float.  Each sublayer's output is not added at once:
it is handed on as ``delta`` and added inside the next norm's kernel (one pass over
``h`` instead of two), so a block takes and returns ``(h, delta)``.

With ``residual_scale`` m every sublayer's output joins the stream times that constant,
``h = h + m * mixer(norm_1(h))``: the output travels as a ``K.PendingNorm`` without a weight and
the next norm's kernel multiplies in float while it adds.  ``has_feed_forward`` False: the
first line only.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import PartSpec, build_part, is_replayable, register_part


class PreNormBlock:
    def __init__(self, norm: PartSpec, mixer_norm_name: str = "input_layernorm",
                 feed_forward_norm_name: str = "post_attention_layernorm", residual_scale: float = 1.0,
                 has_feed_forward: bool = True):
        self.has_feed_forward = bool(has_feed_forward)
        self.residual_scale = float(residual_scale)
        self.mixer_norm = build_part("norm", norm)
        self.feed_forward_norm = build_part("norm", norm) if self.has_feed_forward else None
        self.names = (mixer_norm_name, feed_forward_norm_name) if self.has_feed_forward else (mixer_norm_name,)
        self.norms = (self.mixer_norm, self.feed_forward_norm) if self.has_feed_forward else (self.mixer_norm,)

    @property
    def replayable(self) -> bool:
        return all(is_replayable(n) for n in self.norms)

    def tensors(self) -> dict:
        out = {}
        for name, part in zip(self.names, self.norms):
            for k, v in part.tensors().items():
                out[f"{name}.{k}"] = v
        return out

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        for name, part in zip(self.names, self.norms):
            part.bind({k[len(name) + 1:]: v for k, v in tensors.items() if k.startswith(name + ".")}, dtype)

    def _share(self, out):
        """What a sublayer returned, as the next norm takes it."""
        if self.residual_scale != 1.0 or isinstance(out, tuple):       # a pair (rows, float shares) is added there too
            return K.pending_scale(out, self.residual_scale)
        return out.settled() if isinstance(out, K.BiasedOutput) else out

    def forward(self, h, delta, mixer, feed_forward, ctx, mem):
        n = h.shape[0]
        x = _add_norm(self.mixer_norm, h, delta, mixer, n)
        a = self._share(mixer.forward(x, ctx, mem))
        if not self.has_feed_forward:
            return a
        y = _add_norm(self.feed_forward_norm, h, a, feed_forward, n)
        return self._share(feed_forward.forward(y, ctx))


def _add_norm(norm, h, delta, reader, n_rows: int):
    """``norm.add_norm(h, delta)``.  Only where both sides have said so, the norm may hand on
    ``K.UnscaledRows``: a norm part declares ``may_leave_scale = True`` (its ``add_norm`` takes
    ``unscaled_ok``), a reader part answers ``takes_unscaled_rows(rows)``.  Parts that declare
    neither see the plain interface."""
    ask = getattr(reader, "takes_unscaled_rows", None)
    if (getattr(norm, "may_leave_scale", False) and ask is not None and not isinstance(delta, K.PendingNorm)
            and ask(n_rows)):
        return norm.add_norm(h, delta, unscaled_ok=True)
    return norm.add_norm(h, delta)


class SandwichBlock:
    """Every sublayer between two norms:

        h = h + norm_1b(mixer(norm_1(h)));   h = h + norm_2b(feed_forward(norm_2(h)))

    (the second line only for a layer that has a feed-forward).  A sublayer's output is handed on as a
    ``K.PendingNorm`` (the output and the norm weight that belongs to it): the next norm's kernel norms it,
    adds it to the stream and norms the stream in one pass, also across the border of two layers and
    before the head."""

    def __init__(self, norm: PartSpec, has_feed_forward: bool = True,
                 names=("norm1", "norm1b", "norm2", "norm2b")):
        self.has_feed_forward = bool(has_feed_forward)
        self.names = tuple(names) if self.has_feed_forward else tuple(names[:2])
        self.norms = [build_part("norm", norm) for _ in self.names]

    @property
    def replayable(self) -> bool:
        return all(is_replayable(n) for n in self.norms)

    def tensors(self) -> dict:
        out = {}
        for name, part in zip(self.names, self.norms):
            for k, v in part.tensors().items():
                out[f"{name}.{k}"] = v
        return out

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        for name, part in zip(self.names, self.norms):
            part.bind({k[len(name) + 1:]: v for k, v in tensors.items() if k.startswith(name + ".")}, dtype)

    def forward(self, h, delta, mixer, feed_forward, ctx, mem):
        from ..ops import kernels as K

        x = self.norms[0].add_norm(h, delta)
        a = mixer.forward(x, ctx, mem)
        pending = K.pending_norm(a, self.norms[1].weight, self.norms[1].eps)
        if not self.has_feed_forward:
            return pending
        y = self.norms[2].add_norm(h, pending)
        f = feed_forward.forward(y, ctx)
        return K.pending_norm(f, self.norms[3].weight, self.norms[3].eps)


class OutputNormBlock:
    """A norm on every sublayer's OUTPUT only; the sublayers read the stream itself:

        h = h + norm_1(mixer(h));   h = h + norm_2(feed_forward(h))

    (the second line only for a layer that has a feed-forward; a constant factor on the sublayer's share is the
    norm part's ``gain``).  A sublayer's output is handed on as a ``K.PendingNorm``; the kernel that norms it and adds
    it to the float stream also hands the next reader the stream in the activation type."""

    def __init__(self, norm: PartSpec, has_feed_forward: bool = True, names=("norm1", "norm2")):
        self.has_feed_forward = bool(has_feed_forward)
        self.names = tuple(names) if self.has_feed_forward else tuple(names[:1])
        self.norms = [build_part("norm", norm) for _ in self.names]

    @property
    def replayable(self) -> bool:
        return all(is_replayable(n) for n in self.norms)

    def tensors(self) -> dict:
        out = {}
        for name, part in zip(self.names, self.norms):
            for k, v in part.tensors().items():
                out[f"{name}.{k}"] = v
        return out

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        for name, part in zip(self.names, self.norms):
            part.bind({k[len(name) + 1:]: v for k, v in tensors.items() if k.startswith(name + ".")}, dtype)

    def _stream(self, h, delta):
        """h += (what ``delta`` still owes the stream); returns h in the activation type."""
        from ..ops import kernels as K

        if delta is None:
            return K.cast_rows(h, self.dtype)
        if not isinstance(delta, K.PendingNorm):
            raise TypeError("this arrangement follows layers that hand on a sublayer's output with its norm")
        out = torch.empty(h.shape, dtype=self.dtype, device=h.device)
        K.postnorm_add_rmsnorm(h, delta.y, delta.parts, delta.weight, delta.eps, None, out, bias=delta.bias,
                               plain_scale=delta.scale)
        return out

    def forward(self, h, delta, mixer, feed_forward, ctx, mem):
        from ..ops import kernels as K

        a = mixer.forward(self._stream(h, delta), ctx, mem)
        pending = K.pending_norm(a, self.norms[0].weight, self.norms[0].eps)
        if not self.has_feed_forward:
            return pending
        f = feed_forward.forward(self._stream(h, pending), ctx)
        return K.pending_norm(f, self.norms[1].weight, self.norms[1].eps)


class ParallelBlock:
    """One norm whose output both sublayers read, their outputs joining the stream together, and an optional
    per-layer token input behind them (``parts/token_input.py``):

        u = norm_1(h);   h = h + (mixer(u) + feed_forward(u));   h = h + norm_t(token_input(h))

    (the feed-forward and the token input are optional).  The sublayers' outputs are added to the float stream by
    one kernel that also hands the token input the stream in the activation type; the token input's output is
    handed on as a ``K.PendingNorm`` with its own norm weight (a plain RMS norm), so the next layer's norm (or the
    final one) does both norms and the residual step in one pass."""

    def __init__(self, norm: PartSpec, has_feed_forward: bool = True, token_input: PartSpec | None = None,
                 norm_name: str = "norm1", token_input_prefix: str = "side."):
        self.has_feed_forward = bool(has_feed_forward)
        self.norm = build_part("norm", norm)
        self.norm_name, self.token_prefix = norm_name, token_input_prefix
        self.token_input = build_part("token_input", token_input) if token_input is not None else None

    @property
    def replayable(self) -> bool:
        return is_replayable(self.norm) and (self.token_input is None or is_replayable(self.token_input))

    def tensors(self) -> dict:
        out = {f"{self.norm_name}.{k}": v for k, v in self.norm.tensors().items()}
        if self.token_input is not None:
            out.update({self.token_prefix + k: v for k, v in self.token_input.tensors().items()})
        return out

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        name = self.norm_name + "."
        self.norm.bind({k[len(name):]: v for k, v in tensors.items() if k.startswith(name)}, dtype)
        if self.token_input is not None:
            p = self.token_prefix
            self.token_input.bind({k[len(p):]: v for k, v in tensors.items() if k.startswith(p)}, dtype)

    def forward(self, h, delta, mixer, feed_forward, ctx, mem):
        u = self.norm.add_norm(h, delta)
        a = mixer.forward(u, ctx, mem)
        f = feed_forward.forward(u, ctx) if self.has_feed_forward else None
        if self.token_input is None:
            K.add_outputs(h, a, f)
            return None
        x = K.add_outputs(h, a, f, out_dtype=self.dtype)
        y = self.token_input.forward(x, ctx)
        return K.pending_norm(y, self.token_input.norm_weight, self.token_input.eps)


register_part("block", "prenorm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "output_norm", OutputNormBlock)
register_part("block", "sandwich", SandwichBlock)
