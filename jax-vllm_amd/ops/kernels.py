"""Typed Python entry points of the HIP kernels.

Every wrapper checks on the host that the operands have the device, type,
contiguity and shapes that the kernel and its grid assume, then launches on
torch's current stream.  There is no other implementation behind these
functions: a missing library raises ``KernelLibraryError``.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

from . import library

_SUFFIX = {torch.bfloat16: "bf16", torch.float32: "f32"}


class KernelArgumentError(ValueError):
    """An operand does not have the shape, type or layout the kernel needs."""


def _suffix(dtype: torch.dtype) -> str:
    try:
        return _SUFFIX[dtype]
    except KeyError:
        raise KernelArgumentError(f"kernels take bfloat16 or float32, not {dtype}") from None


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelArgumentError(msg)


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operands must live on the GPU")
            _need(t.is_contiguous(), "kernel operands must be contiguous")


def _check(code: int, name: str) -> None:
    if code == 1:   # hipErrorInvalidValue: what an entry point returns for sizes it is not built for
        raise KernelArgumentError(f"{name}: the kernel library refused these sizes or this block shape")
    if code != 0:
        raise RuntimeError(f"{name}: HIP error {code}")


def _i32(t, name: str, n: int | None = None) -> None:
    _need(t.dtype == torch.int32, f"{name} must be int32")
    if n is not None:
        _need(t.numel() == n, f"{name} must have {n} entries, has {t.numel()}")


def _f32(t, name: str, n: int | None = None) -> None:
    _need(t.dtype == torch.float32, f"{name} must be float32")
    if n is not None:
        _need(t.numel() == n, f"{name} must have {n} entries, has {t.numel()}")


# --------------------------------------------------------------------------- embedding
def embedding(h: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> None:
    """h[t] = float(table[ids[t]]).  An id outside [0, rows) reads nothing and makes its row NaN."""
    _dev(h, table, ids)
    n, hidden = h.shape
    _f32(h, "h")
    _i32(ids, "ids", n)
    _need(table.dim() == 2 and table.shape[1] == hidden, "table width differs from h")
    fn = getattr(library.core(), f"jv_embedding_{_suffix(table.dtype)}")
    _check(fn(_ptr(h), _ptr(table), _ptr(ids), c_int(n), c_int(hidden), c_int(table.shape[0]), _stream()), "embedding")


# --------------------------------------------------------------------------- norms
def add_rmsnorm(h, delta, weight, out, eps: float, rows=None) -> None:
    """Residual add and RMSNorm in one pass.

    Without ``rows``: h += delta (in place, float), out = norm(h) * weight for every row.
    With ``rows`` (int32 indices): out[i] = norm(h[rows[i]] + delta[rows[i]]) * weight and
    h is left as it is.  ``delta`` may be None, or a float32 stack [parts, rows of h, hidden] of
    partial products (``linear(..., partial_ok=True)``), which are added in their order.
    """
    _dev(h, delta, weight, out, rows)
    _f32(h, "h")
    hidden = h.shape[-1]
    _f32(weight, "weight", hidden)
    n_out = out.shape[0]
    _need(out.shape[-1] == hidden, "out width differs from h")
    if rows is None:
        _need(n_out == h.shape[0], "out must have one row per row of h")
    else:
        _i32(rows, "rows", n_out)
    if delta is not None and delta.dim() == 3:
        _need(delta.dtype == torch.float32 and delta.shape[1:] == h.shape and delta.shape[0] <= 4,
              "partial products must be float32 [parts <= 4, *h.shape]")
        _need(hidden % 4 == 0 and hidden <= PARTIAL_SUM_MAX_WIDTH, "partial products need a width that is a multiple of 4, at most 8192")
        fn = getattr(library.core(), f"jv_add_rmsnorm_parts_{_suffix(out.dtype)}")
        _check(
            fn(_ptr(h), _ptr(delta), c_int(delta.shape[0]), c_longlong(delta.stride(0)), _ptr(weight), _ptr(out),
               _ptr(rows), c_int(n_out), c_int(hidden), c_float(eps), _stream()),
            "add_rmsnorm",
        )
        return
    if delta is not None:
        _need(delta.shape == h.shape and delta.dtype == out.dtype, "delta must match h's shape and out's type")
    fn = getattr(library.core(), f"jv_add_rmsnorm_{_suffix(out.dtype)}")
    _check(
        fn(_ptr(h), _ptr(delta), _ptr(weight), _ptr(out), _ptr(rows), c_int(n_out), c_int(hidden),
           c_float(eps), _stream()),
        "add_rmsnorm",
    )


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out=None) -> torch.Tensor:
    """RMSNorm over the last axis of a contiguous tensor."""
    out = torch.empty_like(x) if out is None else out
    _dev(x, weight, out)
    n = x.shape[-1]
    _f32(weight, "weight", n)
    _need(out.shape == x.shape and out.dtype == x.dtype, "out must match x")
    fn = getattr(library.core(), f"jv_rmsnorm_{_suffix(x.dtype)}")
    _check(fn(_ptr(out), _ptr(x), _ptr(weight), c_longlong(x.numel() // n), c_int(n), c_float(eps), _stream()),
           "rmsnorm")
    return out


UNSCALED_SHARE = 512          # columns of a row per block of the un-normalised residual step
UNSCALED_MAX_SHARES = 16      # shares of a row's sum of squares that the products' epilogue adds


class UnscaledRows:
    """Rows ``x = h * weight`` in bfloat16 whose RMSNorm scale is still to be applied: row m of what a
    product with them gives has to be multiplied by ``rsqrt(sum(ssq[m]) / width + eps)`` (the scale of
    a row commutes with the product).  ``linear`` does that in the epilogue of its streaming kernels."""

    def __init__(self, x: torch.Tensor, ssq: torch.Tensor, width: int, eps: float):
        self.x, self.ssq, self.width, self.eps = x, ssq, int(width), float(eps)   # ssq [rows, 16], width / 512 of them used
        self.shares = self.width // UNSCALED_SHARE

    shape = property(lambda self: self.x.shape)
    dtype = property(lambda self: self.x.dtype)
    device = property(lambda self: self.x.device)


def unscaled_rows_possible(dtype, n_rows: int, hidden: int) -> bool:
    return (dtype == torch.bfloat16 and 0 < n_rows <= SKINNY_AUTO_ROWS and hidden % UNSCALED_SHARE == 0
            and hidden // UNSCALED_SHARE <= UNSCALED_MAX_SHARES)


def add_parts_unscaled(h: torch.Tensor, parts: torch.Tensor, weight: torch.Tensor, eps: float) -> "UnscaledRows":
    """h += parts[0] + parts[1] + ... (in that order, in place, float); returns the rows h * weight in
    bfloat16, NOT normalised, with the shares of each row's sum of squares: the residual step of a
    decode step shared out to hidden / 512 blocks a row instead of one (the norm's reduction would
    need the whole row in one block)."""
    _dev(h, parts, weight)
    _f32(h, "h")
    n, hidden = h.shape
    _f32(weight, "weight", hidden)
    _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[1:] == h.shape and 1 <= parts.shape[0] <= 4,
          "partial products must be float32 [parts <= 4, *h.shape]")
    _need(unscaled_rows_possible(torch.bfloat16, n, hidden), "at most 16 rows of a width that is a multiple of 512, at most 8192")
    xg = torch.empty((n, hidden), dtype=torch.bfloat16, device=h.device)
    ssq = torch.empty((n, UNSCALED_MAX_SHARES), dtype=torch.float32, device=h.device)    # hidden / 512 of a row's 16 are written
    _check(library.core().jv_add_parts_unscaled_bf16(_ptr(h), _ptr(parts), c_int(parts.shape[0]), c_longlong(parts.stride(0)),
                                                     _ptr(weight), _ptr(xg), _ptr(ssq), c_int(n), c_int(hidden), _stream()),
           "add_parts_unscaled")
    return UnscaledRows(xg, ssq, hidden, eps)


def cast_rows(x: torch.Tensor, dtype: torch.dtype, rows=None) -> torch.Tensor:
    """Copy (selected) rows of a float matrix into a new matrix of ``dtype``."""
    _dev(x, rows)
    _f32(x, "x")
    n_out = x.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, "rows")
    out = torch.empty((n_out, x.shape[1]), dtype=dtype, device=x.device)
    fn = getattr(library.core(), f"jv_cast_rows_{_suffix(dtype)}")
    _check(fn(_ptr(out), _ptr(x), _ptr(rows), c_int(n_out), c_int(x.shape[1]), _stream()), "cast_rows")
    return out


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """y[..., c] += bias[c] in place, for what ``linear`` returned: rows [M, N], or a float stack [parts, M, N]
    of partial products, of which the first takes the bias."""
    _dev(y, bias)
    rows = y[0] if y.dim() == 3 else y
    _need(rows.dim() == 2 and rows.is_contiguous() and bias.is_contiguous(), "y must be contiguous rows")
    _f32(bias, "bias", rows.shape[1])
    fn = getattr(library.core(), f"jv_add_bias_{_suffix(rows.dtype)}")
    _check(fn(_ptr(rows), _ptr(bias), c_longlong(rows.shape[0]), c_int(rows.shape[1]), _stream()), "add_bias")


PLAIN_ACTIVATIONS = {None: 0, "silu": 1, "gelu_tanh": 2, "gelu": 3, "tanh": 4}     # ids of act in y = act(x + bias); "gelu" is the erf form


def bias_act(y: torch.Tensor, bias, activation) -> None:
    """y[r, c] = act(y[r, c] + bias[c]) in place for contiguous rows; ``bias`` float32 or None, ``activation`` one of
    ``PLAIN_ACTIVATIONS`` (None: the bias alone); computed in float."""
    _dev(y, bias)
    _need(y.dim() == 2, "y must be rows")
    _need(activation in PLAIN_ACTIVATIONS, f"no kernel for the activation {activation!r}: there are {sorted(map(str, PLAIN_ACTIVATIONS))}")
    if bias is not None:
        _f32(bias, "bias", y.shape[1])
    fn = getattr(library.core(), f"jv_bias_act_{_suffix(y.dtype)}")
    _check(fn(_ptr(y), _ptr(bias), c_longlong(y.shape[0]), c_int(y.shape[1]), c_int(PLAIN_ACTIVATIONS[activation]), _stream()),
           "bias_act")


def scaled_sum(out: torch.Tensor, y, scale: float) -> None:
    """out = scale * y as float, where ``y`` is what a sublayer returned: rows of the activation type, a float stack
    [P, rows, width] of partial results (added in order), or a pair (rows or None, stack or None)."""
    rows, parts = split_sublayer_output(y)
    _dev(out, rows, parts)
    _f32(out, "out")
    _need(rows is not None or parts is not None, "nothing to add")
    if rows is not None:
        _need(rows.shape == out.shape, "rows must match out's shape")
    if parts is not None:
        _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[1:] == out.shape, "parts must be float32 [P, *out.shape]")
    kind = rows.dtype if rows is not None else torch.float32
    fn = getattr(library.core(), f"jv_scaled_sum_{_suffix(kind)}")
    _check(fn(_ptr(out), _ptr(rows), _ptr(parts), c_int(0 if parts is None else parts.shape[0]),
              c_longlong(0 if parts is None else parts.stride(0)), c_longlong(out.numel()), c_float(scale), _stream()), "scaled_sum")


def embedding_pair(h: torch.Tensor, table: torch.Tensor, pair, ids: torch.Tensor, prev: torch.Tensor,
                   buckets: int, mul_prev: int, mul_cur: int, scale: float = 1.0) -> None:
    """h[t] = scale * float(table[ids[t]]) + float(pair[r]) with r = (prev[t] * mul_prev + ids[t] * mul_cur) mod buckets,
    or r = buckets (the last row of ``pair``) where prev[t] < 0: a sequence's first token.  ``pair`` None: the scaled
    row alone."""
    _dev(h, table, pair, ids, prev)
    n, hidden = h.shape
    _f32(h, "h")
    _i32(ids, "ids", n)
    _i32(prev, "prev", n)
    _need(table.dim() == 2 and table.shape[1] == hidden and table.is_contiguous(), "table width differs from h")
    _need(pair is None or (pair.shape == (buckets + 1, hidden) and pair.dtype == table.dtype and pair.is_contiguous()),
          "the pair table must be [buckets + 1, hidden] of the table's type")
    _need(buckets > 0 and 0 <= mul_prev < 2 ** 31 and 0 <= mul_cur < 2 ** 31, "buckets must be positive, the multipliers below 2^31")
    fn = getattr(library.core(), f"jv_embedding_pair_{_suffix(table.dtype)}")
    _check(fn(_ptr(h), _ptr(table), _ptr(pair), _ptr(ids), _ptr(prev), c_int(n), c_int(hidden), c_int(table.shape[0]),
              c_longlong(buckets), c_longlong(mul_prev), c_longlong(mul_cur), c_float(scale), _stream()), "embedding_pair")


def add_outputs(h: torch.Tensor, a, b=None, out_dtype=None):
    """h += a + b in the float residual stream (the sum of the two first, then the stream), where ``a`` and ``b`` are
    what two sublayers returned: rows of the activation type, a float stack [P, rows, width] of partial results
    (added in order), a pair (rows or None, stack or None), or None.  With ``out_dtype`` returns the new h in
    that type."""
    ra, pa = split_sublayer_output(a) if a is not None else (None, None)
    rb, pb = split_sublayer_output(b) if b is not None else (None, None)
    _dev(h, ra, pa, rb, pb)
    _f32(h, "h")
    _need(h.is_contiguous(), "h must be contiguous")
    kinds = {t.dtype for t in (ra, rb) if t is not None}
    _need(len(kinds) <= 1 and (out_dtype is None or not kinds or kinds == {out_dtype}), "rows and the output must have one type")
    kind = next(iter(kinds), out_dtype or torch.float32)
    for t in (ra, rb):
        _need(t is None or (t.shape == h.shape and t.is_contiguous()), "rows must match h's shape")
    for t in (pa, pb):
        _need(t is None or (t.dtype == torch.float32 and t.dim() == 3 and t.shape[1:] == h.shape and t[0].is_contiguous()),
              "parts must be float32 [P, *h.shape]")
    out = torch.empty(h.shape, dtype=out_dtype, device=h.device) if out_dtype is not None else None
    n = h.numel()
    strides = [t.stride(0) if t is not None else 0 for t in (pa, pb)]
    vec = h.shape[1] % 4 == 0 and all(s % 4 == 0 for s in strides) and all(
        t is None or t.data_ptr() % 16 == 0 for t in (h, ra, pa, rb, pb, out))
    fn = getattr(library.core(), f"jv_add_outputs_{_suffix(kind)}")
    _check(fn(_ptr(h), _ptr(ra), _ptr(pa), c_int(0 if pa is None else pa.shape[0]), c_longlong(strides[0]),
              _ptr(rb), _ptr(pb), c_int(0 if pb is None else pb.shape[0]), c_longlong(strides[1]), _ptr(out),
              c_longlong(n), c_int(1 if vec else 0), _stream()), "add_outputs")
    return out


def token_gate_mul(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, offset: int, activation="gelu_tanh") -> None:
    """z[t, c] = act(z[t, c]) * table[ids[t], offset + c] in place for contiguous rows z [n, dim]; ``activation`` one
    of ``PLAIN_ACTIVATIONS``, computed in float."""
    _dev(z, table, ids)
    n, dim = z.shape
    _i32(ids, "ids", n)
    _need(z.is_contiguous() and table.dim() == 2 and table.is_contiguous() and table.dtype == z.dtype,
          "z and the table must be contiguous and of one type")
    _need(0 <= offset and offset + dim <= table.shape[1], "the columns lie outside the table")
    _need(activation in PLAIN_ACTIVATIONS, f"no kernel for the activation {activation!r}")
    fn = getattr(library.core(), f"jv_token_gate_mul_{_suffix(z.dtype)}")
    _check(fn(_ptr(z), _ptr(table), _ptr(ids), c_longlong(n), c_int(dim), c_int(table.shape[1]), c_int(offset),
              c_int(table.shape[0]), c_int(PLAIN_ACTIVATIONS[activation]), _stream()), "token_gate_mul")


def sigmoid_gate_heads(o: torch.Tensor, gate: torch.Tensor, heads: int, dv: int, dp: int) -> None:
    """o[t, h * dp + i] *= sigmoid(gate[t, h * dv + i]) for i < dv, in place: o [n, heads * dp] contiguous, ``gate`` a
    [n, heads * dv] view with unit column stride (any row stride) of the same type."""
    _dev(o)
    n = o.shape[0]
    _need(o.is_contiguous() and o.shape == (n, heads * dp) and dp >= dv, "o must be [n, heads * dp]")
    _need(gate.is_cuda and gate.dtype == o.dtype and gate.shape == (n, heads * dv) and (n == 0 or gate.stride(1) == 1),
          "gate must be a [n, heads * dv] view with unit column stride")
    fn = getattr(library.core(), f"jv_sigmoid_gate_heads_{_suffix(o.dtype)}")
    _check(fn(_ptr(o), _ptr(gate), c_longlong(gate.stride(0)), c_longlong(n), c_int(heads), c_int(dv), c_int(dp), _stream()),
           "sigmoid_gate_heads")


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap) in place (float32, contiguous)."""
    _dev(logits)
    _f32(logits, "logits")
    _need(logits.is_contiguous() and cap > 0, "contiguous logits and a positive cap")
    _check(library.core().jv_softcap_f32(_ptr(logits), c_longlong(logits.numel()), c_float(cap), _stream()), "softcap")
    return logits


# --------------------------------------------------------------------------- activation
GATE_ACTIVATIONS = {"silu": 1, "gelu_tanh": 2}      # the kernels' ids of act in y = act(gate) * up


def _gate_act_id(name) -> int:
    _need(name in GATE_ACTIVATIONS, f"no kernel for the gate activation {name!r}: there are {sorted(GATE_ACTIVATIONS)}")
    return GATE_ACTIVATIONS[name]


def gated_mul(gate_up: torch.Tensor, out=None, interleaved: bool = False, activation: str = "silu") -> torch.Tensor:
    """out[t, j] = act(gate) * up for gate_up of width 2 I: gate = gate_up[t, j], up =
    gate_up[t, I + j], or with ``interleaved`` gate = gate_up[t, 2j], up = gate_up[t, 2j + 1];
    ``activation`` is one of ``GATE_ACTIVATIONS``, computed in float."""
    _dev(gate_up)
    n, two_i = gate_up.shape
    _need(two_i % 2 == 0, "gate_up must have an even width")
    inter = two_i // 2
    if out is None:
        out = torch.empty((n, inter), dtype=gate_up.dtype, device=gate_up.device)
    _dev(out)
    _need(out.shape == (n, inter) and out.dtype == gate_up.dtype, "out must be [tokens, I] of gate_up's type")
    fn = getattr(library.core(), f"jv_gated_mul_{_suffix(gate_up.dtype)}")
    _check(fn(_ptr(out), _ptr(gate_up), c_longlong(n), c_int(inter), c_int(1 if interleaved else 0),
              c_int(_gate_act_id(activation)), _stream()), "gated_mul")
    return out


def _check_pages(k_pages, v_pages, dtype, nkv, page_size, head_dim) -> None:
    _need(k_pages.dtype == dtype and v_pages.dtype == dtype, "cache pages must have the activation type")
    _need(k_pages.dim() == 4 and tuple(k_pages.shape[1:]) == (nkv, page_size, head_dim),
          "key pages must be [pages, nkv, page_size, D]")
    _need(v_pages.dim() == 4 and tuple(v_pages.shape[1:]) == (nkv, head_dim, page_size),
          "value pages must be [pages, nkv, D, page_size]")
    _need(k_pages.shape[0] == v_pages.shape[0], "key and value pages differ in number")


# --------------------------------------------------------------------------- attention input
def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, out=None) -> torch.Tensor:
    """float32 [tokens, 2 * half]: cos(pos * inv_freq) then sin(pos * inv_freq), angles in float."""
    _dev(positions, inv_freq, out)
    n, half = positions.numel(), inv_freq.numel()
    _i32(positions, "positions")
    _f32(inv_freq, "inv_freq")
    if out is None:
        out = torch.empty((n, 2 * half), dtype=torch.float32, device=positions.device)
    _need(out.shape == (n, 2 * half) and out.dtype == torch.float32, "table must be float32 [tokens, 2 * half]")
    _check(library.core().jv_rope_table(_ptr(out), _ptr(positions), _ptr(inv_freq), c_int(n), c_int(half),
                                        _stream()), "rope_table")
    return out


def rope_takes_parts(dtype, head_dim: int, interleaved: bool, rotary_dim: int, rotated: bool) -> bool:
    """Whether ``qk_norm_rope_write`` takes its input as float partial products (``parts``)."""
    return (dtype == torch.bfloat16 and head_dim in (128, 256) and not interleaved
            and (not rotated or (rotary_dim % 128 == 0 and rotary_dim > 0)))


def qk_norm_rope_write(qkv, slot_mapping, q_weight, k_weight, eps, cos_sin, rotary_dim, interleaved,
                       k_pages, v_pages, page_size, nq, nkv, head_dim, parts=None) -> None:
    """Per-head q/k RMSNorm (if weights given), rotation (if a ``rope_table`` is given), q in
    place, k and v into their pages (if pages given): K [pages, nkv, page_size, D], V transposed
    [pages, nkv, D, page_size].  With ``parts`` (float32 [2..4, tokens, (nq + 2 nkv) * D], see
    ``linear(..., partial_ok=True)``) the input is the sum of the parts, added in order, and
    ``qkv`` only receives the q heads."""
    _dev(qkv, slot_mapping, q_weight, k_weight, cos_sin, k_pages, v_pages, parts)
    n = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nq + 2 * nkv) * head_dim, "qkv must be [tokens, (nq + 2 nkv) * D]")
    _need(head_dim <= 512, "head size above 512 is not supported by the rotation kernel")
    if q_weight is not None:
        _f32(q_weight, "q_weight", head_dim)
    if k_weight is not None:
        _f32(k_weight, "k_weight", head_dim)
    if cos_sin is not None:
        _need(rotary_dim % 2 == 0 and 0 < rotary_dim <= head_dim, "rotary_dim must be even and at most D")
        _f32(cos_sin, "cos_sin", n * rotary_dim)
    if k_pages is not None:
        _i32(slot_mapping, "slot_mapping", n)
        _check_pages(k_pages, v_pages, qkv.dtype, nkv, page_size, head_dim)
    if parts is not None:
        _need(rope_takes_parts(qkv.dtype, head_dim, interleaved, rotary_dim, cos_sin is not None),
              "partial products are taken for bfloat16, head size 128 or 256, half-split pairing, full rotation")
        _need(parts.dtype == torch.float32 and parts.dim() == 3 and 2 <= parts.shape[0] <= 4
              and parts.shape[1:] == qkv.shape, "parts must be float32 [2..4, tokens, (nq + 2 nkv) * D]")
        _check(
            library.core().jv_qk_norm_rope_write_parts_bf16(
                _ptr(qkv), _ptr(parts), c_int(parts.shape[0]), c_longlong(parts.stride(0)),
                _ptr(slot_mapping if k_pages is not None else None), _ptr(q_weight), _ptr(k_weight), c_float(eps),
                _ptr(cos_sin), c_int(rotary_dim if cos_sin is not None else 0), _ptr(k_pages), _ptr(v_pages),
                c_int(page_size), c_int(n), c_int(nq), c_int(nkv), c_int(head_dim), _stream()),
            "qk_norm_rope_write",
        )
        return
    fn = getattr(library.core(), f"jv_qk_norm_rope_write_{_suffix(qkv.dtype)}")
    _check(
        fn(_ptr(qkv), _ptr(slot_mapping if k_pages is not None else None), _ptr(q_weight), _ptr(k_weight),
           c_float(eps), _ptr(cos_sin), c_int(rotary_dim if cos_sin is not None else 0),
           c_int(1 if interleaved else 0), _ptr(k_pages), _ptr(v_pages), c_int(page_size), c_int(n),
           c_int(nq), c_int(nkv), c_int(head_dim), _stream()),
        "qk_norm_rope_write",
    )


def padded_head_dim(dk: int, dv: int) -> int:
    """The one head size under which keys of ``dk`` and values of ``dv`` elements are cached (zeros behind them):
    the next multiple of 16, which the matrix-core attention kernels are built for."""
    return -(-max(int(dk), int(dv)) // 16) * 16


def attn_prepare_wide(qkv, bias, q_weight, k_weight, eps: float, cos_sin, rot_dims: int, slot_mapping, k_pages, v_pages,
                      page_size: int, nq: int, nkv: int, dk: int, dv: int, dp: int, v_scale: float = 1.0,
                      norm_per_head: bool = False, values_are_keys: bool = False, positions=None,
                      q_temperature: "tuple | None" = None) -> torch.Tensor:
    """Attention input whose key and value sizes differ, whose q/k norm spans the whole projection, or whose rows
    carry more than q, k and v.  ``qkv`` rows
    begin with [q: nq * dk | k: nkv * dk | v: nkv * dv] (further columns are left alone); ``bias`` (float32, that width) is added first; with
    ``q_weight`` [nq * dk] and ``k_weight`` [nkv * dk] q and k are RMS-normed over all their columns at once (with
    ``norm_per_head``: every head on its own, with weights [dk] shared by the heads); the
    first ``rot_dims`` elements of every q and k head turn by ``cos_sin`` (``rope_table``); v is multiplied by
    ``v_scale``.  ``values_are_keys``: the rows hold [q | k] only and the values are the k columns as projected (before
    bias-free norm and rotation; needs dv == dk and no whole-projection norm).  ``q_temperature`` (coef, every) with
    ``positions`` (int32 [n]): q at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).  Returns q as [n, nq * dp] with every head padded with zeros to ``dp``; keys go to
    [pages, nkv, page_size, dp], values to [pages, nkv, dp, page_size] (their pad is never written)."""
    _dev(qkv, bias, q_weight, k_weight, cos_sin, slot_mapping, k_pages, v_pages)
    n, ld = qkv.shape
    v_off = nq * dk if values_are_keys else (nq + nkv) * dk
    width = v_off + nkv * dv
    _need(not values_are_keys or (dv == dk and (q_weight is None or norm_per_head)),
          "values that are the keys have the keys' size, and the norm is per head or none")
    _need(qkv.dim() == 2 and ld >= width and qkv.is_contiguous(), "qkv rows must begin with nq * dk + nkv * dk + nkv * dv columns")
    coef, every = (0.0, 1)
    if q_temperature is not None:
        coef, every = float(q_temperature[0]), int(q_temperature[1])
        _need(every > 0 and positions is not None and (q_weight is None or norm_per_head),
              "a query temperature needs positions, a positive period and a per-head norm or none")
        _dev(positions)
        _i32(positions, "positions", n)
    _need(dp >= max(dk, dv), "the padded head size must hold keys and values")
    if bias is not None:
        _f32(bias, "bias", width)
    _need((q_weight is None) == (k_weight is None), "q and k are normed together or not at all")
    if q_weight is not None:
        _f32(q_weight, "q_weight", dk if norm_per_head else nq * dk)
        _f32(k_weight, "k_weight", dk if norm_per_head else nkv * dk)
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= dk, "the rotated size must be even and at most the key size")
    if rot_dims:
        _f32(cos_sin, "cos_sin", n * rot_dims)
    if k_pages is not None:
        _i32(slot_mapping, "slot_mapping", n)
        _check_pages(k_pages, v_pages, qkv.dtype, nkv, page_size, dp)
    q = torch.empty((n, nq * dp), dtype=qkv.dtype, device=qkv.device)
    fn = getattr(library.core(), f"jv_attn_prepare_wide_{_suffix(qkv.dtype)}")
    _check(fn(_ptr(q), _ptr(qkv), c_longlong(ld), _ptr(bias), _ptr(q_weight), _ptr(k_weight), c_float(eps),
              _ptr(cos_sin if rot_dims else None), c_int(rot_dims), _ptr(slot_mapping if k_pages is not None else None),
              _ptr(k_pages), _ptr(v_pages), c_int(page_size), c_int(n), c_int(nq), c_int(nkv), c_int(dk), c_int(dv),
              c_int(dp), c_float(v_scale), c_int(1 if norm_per_head else 0), c_longlong(v_off),
              _ptr(positions if q_temperature is not None else None), c_float(coef), c_int(every), _stream()), "attn_prepare_wide")
    return q


# --------------------------------------------------------------------------- attention
def paged_attention_generic(out, q, q_row_stride, k_pages, v_pages, block_tables, token_req, positions,
                            nq, nkv, head_dim, scale, window=0, sinks=None) -> None:
    """Causal attention of every token over its request's pages (generic float-math kernel).

    ``q`` is any tensor whose row t holds the q heads at [t * q_row_stride + h * D].  ``sinks`` (float32 [nq]):
    exp(sinks[h]) joins every row's softmax denominator (a term without key and value, not scaled)."""
    _dev(out, q, k_pages, v_pages, block_tables, token_req, positions, sinks)
    if sinks is not None:
        _f32(sinks, "sinks", nq)
    n = out.shape[0]
    _need(out.shape == (n, nq * head_dim) and out.dtype == q.dtype, "out must be [tokens, nq * D] of q's type")
    _need(q.numel() >= (n - 1) * q_row_stride + nq * head_dim if n else True, "q is too small for its stride")
    _need(nkv > 0 and nq % nkv == 0, "q heads must be a multiple of kv heads")
    _need(head_dim <= 640, "head size above 640 is not supported")
    page_size = k_pages.shape[2]
    _check_pages(k_pages, v_pages, q.dtype, nkv, page_size, head_dim)
    _need(block_tables.dim() == 2, "block_tables must be [requests, pages]")
    _i32(block_tables, "block_tables")
    _i32(token_req, "token_req", n)
    _i32(positions, "positions", n)
    fn = getattr(library.core(), f"jv_paged_attention_generic_{_suffix(q.dtype)}")
    _check(
        fn(_ptr(out), _ptr(q), c_longlong(q_row_stride), _ptr(k_pages), _ptr(v_pages), _ptr(block_tables),
           c_int(block_tables.shape[1]), _ptr(token_req), _ptr(positions), c_int(page_size), c_int(n),
           c_int(nq), c_int(nkv), c_int(head_dim), c_float(scale), c_int(window or 0), _ptr(sinks), _stream()),
        "paged_attention_generic",
    )


# --------------------------------------------------------------------------- matrix products
def gemm_f32(a: torch.Tensor, w: torch.Tensor, out=None) -> torch.Tensor:
    """out = a @ w.T in true 32-bit (float FMA).  a [M, K], w [N, K], both row-major."""
    _dev(a, w)
    _f32(a, "a")
    _f32(w, "w")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k, f"inner sizes differ: {k} and {w.shape[1]}")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    _dev(out)
    _need(out.shape == (m, n) and out.dtype == torch.float32, "out must be float32 [M, N]")
    fn = library.core().jv_gemm_f32
    _check(fn(_ptr(out), _ptr(a), _ptr(w), c_int(m), c_int(n), c_int(k), c_longlong(k), c_longlong(k),
              c_longlong(n), _stream()), "gemm_f32")
    return out


SKINNY_MAX_ROWS = 64
SKINNY_AUTO_ROWS = 16   # up to here ``linear`` prefers the streaming kernel to the library
SKINNY_LARGE_MATRIX = 40_000_000    # elements; see streaming_plan
PARTIAL_SUM_MAX_WIDTH = 8192        # widest row whose partial products the norm kernel adds
PARTIAL_BLOCKS = 1024               # a streaming product wants about this many blocks
PARTIAL_SHAPE = (-1, 4, 4)          # x resident in LDS, phases of 512 columns: for inner sizes the staying blocks do not cover


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, out_dtype=torch.bfloat16, gate_pairs: "str | None" = None,
                block_shape=(0, 0, 0), out=None, ksplit: int = 1, row_scale: "UnscaledRows | None" = None) -> torch.Tensor:
    """x @ w.T for at most 64 rows of bfloat16 x against bfloat16 w [N, K]: the weight-streaming
    product of decode steps.  With ``gate_pairs`` (one of ``GATE_ACTIVATIONS``) the rows of w alternate gate
    and up rows and the result is act(x.w[2j]) * (x.w[2j+1]), bfloat16 [M, N/2].  Output bfloat16 or float32.
    ``block_shape``: (row tiles, K slices, MFMA steps per iteration) of a block, zeros: chosen
    from the shape; (-1, waves, pieces) selects the organisation with x resident in LDS;
    (-2, blocks, pieces) the one with blocks that stay and keep x in registers (at most 16 rows,
    inner size at most 256 * pieces).
    ``ksplit`` > 1 (that organisation, float32 output): the inner size is shared out to so many
    blocks per row tile and the result is [ksplit, M, N], partial products to be added in order.
    ``row_scale`` (blocks that stay only): x is ``row_scale.x``, un-normalised rows, and every output
    row (of every partial product) is multiplied by its norm's scale."""
    _dev(x, w, out)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny takes bfloat16")
    m = x.shape[0]
    n, k = w.shape
    _need(x.dim() == 2 and x.shape[1] == k, "inner sizes differ")
    _need(m <= SKINNY_MAX_ROWS, f"gemm_skinny takes at most {SKINNY_MAX_ROWS} rows")
    _need(k % 8 == 0, "the inner size must be a multiple of 8")
    _need(out_dtype in (torch.bfloat16, torch.float32), "output must be bfloat16 or float32")
    _need(block_shape[0] != -2 or ((m <= 16 or (m <= 32 and block_shape[2] in STAY_PIECES_32_ROWS) or block_shape[2] <= 5)
                                   and block_shape[2] in STAY_PIECES
                                   and 256 * block_shape[2] * (ksplit - 1) < k <= 256 * block_shape[2] * ksplit),
          "the organisation with blocks that stay takes at most 16 rows (32 with at most 16 pieces, 64 with at most 5) "
          "and an inner size of ksplit * 256 * pieces at most")
    _need(not gate_pairs or (out_dtype == torch.bfloat16 and n % 2 == 0 and block_shape[0] != -1),
          "the activation epilogue writes bfloat16, needs an even number of rows of w and the chunked organisation")
    _need(ksplit >= 1 and (ksplit == 1 or (block_shape[0] in (-1, -2) and out_dtype == torch.float32
                                           and (m <= 16 or block_shape[0] == -2))),
          "sharing the inner size out needs x resident (at most 16 rows) or blocks that stay, and float32 output")
    n_out = n // 2 if gate_pairs else n
    shape = (m, n_out) if ksplit == 1 else (ksplit, m, n_out)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    _need(out.shape == shape and out.dtype == out_dtype and out.is_contiguous(),
          "out must be [M, N] (or [M, N/2], or [ksplit, M, N]) of the output type")
    common = (_ptr(out), _ptr(x), _ptr(w), c_int(m), c_int(n), c_int(k), c_longlong(x.stride(0)), c_longlong(n_out),
              c_int(1 if out_dtype == torch.float32 else 0), c_int(_gate_act_id(gate_pairs) if gate_pairs else 0),
              c_int(block_shape[0]), c_int(block_shape[1]), c_int(block_shape[2]), c_int(ksplit))
    if row_scale is not None:
        _need(block_shape[0] == -2, "only the blocks that stay scale their output rows")
        _need(row_scale.x is x and row_scale.ssq.is_cuda and row_scale.ssq.dtype == torch.float32
              and row_scale.ssq.is_contiguous() and tuple(row_scale.ssq.shape) == (m, UNSCALED_MAX_SHARES)
              and 1 <= row_scale.shares <= UNSCALED_MAX_SHARES, "row_scale does not belong to x")
        _check(library.core().jv_gemm_skinny_scaled_bf16(*common, _ptr(row_scale.ssq), c_int(row_scale.shares),
                                                         c_int(row_scale.width), c_float(row_scale.eps), _stream()),
               "gemm_skinny")
        return out
    _check(library.core().jv_gemm_skinny_bf16(*common, _stream()), "gemm_skinny")
    return out


def gemm_tile64(x: torch.Tensor, w: torch.Tensor, out_dtype=torch.bfloat16, gate_pairs: "str | None" = None,
                ksplit: int = 1, out=None) -> torch.Tensor:
    """x @ w.T for at most 64 rows of bfloat16 x against bfloat16 w [N, K] with blocks that take 64
    rows of w against all rows of x: the weight-streaming product of decode steps with 17..64
    requests where the library is slow (narrow outputs over a long inner size).  ``gate_pairs`` and ``ksplit`` as in ``gemm_skinny``:
    act(x.w[2j]) * (x.w[2j+1]) as bfloat16 [M, N/2], or float32 partial products [ksplit, M, N] to
    be added in order (every group needs at least one round of 256 columns)."""
    _dev(x, w, out)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_tile64 takes bfloat16")
    m = x.shape[0]
    n, k = w.shape
    _need(x.dim() == 2 and x.shape[1] == k, "inner sizes differ")
    _need(m <= SKINNY_MAX_ROWS, f"gemm_tile64 takes at most {SKINNY_MAX_ROWS} rows")
    _need(k % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0,
          "the inner size and the row stride must be multiples of 8")
    _need(w.is_contiguous(), "w must be contiguous")
    _need(out_dtype in (torch.bfloat16, torch.float32), "output must be bfloat16 or float32")
    _need(not gate_pairs or (out_dtype == torch.bfloat16 and n % 2 == 0 and ksplit == 1),
          "the activation epilogue writes bfloat16, needs an even number of rows of w and an inner size in one piece")
    rounds = -(-k // 256)
    _need(ksplit >= 1 and (ksplit == 1 or (out_dtype == torch.float32 and -(-rounds // ksplit) * (ksplit - 1) < rounds)),
          "sharing the inner size out needs float32 output and a round of 256 columns for every group")
    n_out = n // 2 if gate_pairs else n
    shape = (m, n_out) if ksplit == 1 else (ksplit, m, n_out)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    _need(out.shape == shape and out.dtype == out_dtype and out.is_contiguous(),
          "out must be [M, N] (or [M, N/2], or [ksplit, M, N]) of the output type")
    _check(
        library.core().jv_gemm_tile64_bf16(
            _ptr(out), _ptr(x), _ptr(w), c_int(m), c_int(n), c_int(k), c_longlong(x.stride(0)), c_longlong(n_out),
            c_int(1 if out_dtype == torch.float32 else 0), c_int(_gate_act_id(gate_pairs) if gate_pairs else 0), c_int(ksplit), _stream()),
        "gemm_tile64",
    )
    return out


_cu_count = {}


def compute_units(device) -> int:
    n = _cu_count.get(device)
    if n is None:
        n = _cu_count[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return n


STAY_PIECES = (4, 5, 8, 10, 12, 16, 17, 20)
STAY_PIECES_32_ROWS = (4, 5, 8, 12, 16)      # of these, the ones built for 17..32 rows (two row tiles of x in registers)


def _fit_parts(units: int, parts: int) -> int:
    """The most groups, at most ``parts``, among which ``units`` (phases, chunks) can be shared out
    in equal whole shares without leaving a group empty."""
    while parts > 1 and -(-units // parts) * (parts - 1) >= units:
        parts -= 1
    return parts


def _stay_pieces(k: int, parts: int):
    """Weight pieces per wave with which ``parts`` groups of staying blocks cover an inner size
    of k exactly (each group 8 waves x pieces x 32 columns), or None."""
    for nl in STAY_PIECES:
        if 256 * nl * (parts - 1) < k <= 256 * nl * parts:
            return nl
    return None


TILE64 = (-3, 0, 0)                 # block shape that stands for ``gemm_tile64`` in a plan
TILE64_MIN_SHARE = 3072             # columns a block of gemm_tile64 needs to pay for its start
LIBRARY_MAX_INNER = 12288           # beyond this inner size the library's choice for few rows collapses


def streaming_plan(m: int, n: int, k: int, gate_pairs: bool = False, partial_ok: bool = False, device=None,
                   partial_max_width: int | None = PARTIAL_SUM_MAX_WIDTH):
    """How ``linear`` runs a bfloat16 product at few rows: (block_shape, ksplit) for ``gemm_skinny``
    (``TILE64`` as block shape: for ``gemm_tile64``), or None for the library.  All thresholds are
    measured on MI355X at the matrix shapes of 8B-, 14B- and 32B-class models (pure reads of the
    same bytes: 33 MB 6.5 us, 50 MB 9.1, 101 MB 16.5, 201 MB 33.5).

    * wide matrices (>= 1,024 row tiles), inner size <= 4,096, up to 16 rows: blocks that stay, one per
      compute unit (two for very wide ones), x in registers: 201 MB in 36.7 us at 8 rows, 36.2 at one
      row, against 42 and 38.5 with x staged per block, 44 by the library;
    * narrow matrices whose reader adds partial products, up to 16 rows: the inner size shared out
      to 4 groups so that ~1,000 blocks stream (33 MB: 8.6 us against 11.0 from 256 blocks); staying
      blocks wherever a piece count fits the inner size (4,096 x 12,288 at 8 rows: 20.7 us against 24.9
      with x resident in LDS; 5,120 x 17,408: 35.9 against 40.8; 5,120 x 8,192: 17.9 against 20.0), x
      resident in LDS otherwise (5,120 x 25,600, which would need more than 4 groups);
    * the same at 17..64 rows when every block gets at least 3,072 columns: blocks of 64 rows of w,
      one per compute unit (the feed-forward's second product: 4,096 x 12,288 at 64 rows 30 us
      against the library's 37; 5,120 x 17,408 65 against 131; 5,120 x 25,600 91 against 157);
    * 17..64 rows against narrow matrices with a short inner size (the attention's products): staying
      blocks, one per compute unit, with two to four row tiles of x in registers (up to 8 pieces a
      wave for two, 5 for more), the inner size shared out to 4 groups (4,096 x 4,096: 10.3 us at
      32 rows, 13.2 at 64, against the library's 13.0 and 15.0; 5,120 x 5,120 at 48 rows: 16.5
      against 26.6);
    * 17..32 rows against wide matrices with an inner size of 12 or 16 pieces a wave (gate and up, the output
      embedding): staying blocks with two row tiles of x in registers and W in four slots (24,576 x 4,096
      with the activation at 24 rows 41.9 us, at 32 rows 43.7, against 47.5 and 47.2 by the library and the
      activation kernel; 151,936 x 4,096 at 24 rows 248 against 270);
    * one or two rows against very wide matrices (the output embedding): x resident in LDS (chosen
      inside the kernel library; 1.24 GB in 202 us against 205);
    * 9..16 rows of a large matrix that fits none of these: the library (its wider tiles amortise
      x), unless the inner size is beyond 12,288, where the library needs 113 us for the 178 MB
      that x resident in LDS streams in 45;
    * otherwise x staged chunk by chunk in LDS.
    """
    if k % 8:
        return None
    cus = compute_units(device) if device is not None else 256
    narrow = partial_ok and not gate_pairs and n % 4 == 0 and (partial_max_width is None or n <= partial_max_width)
    if m > SKINNY_AUTO_ROWS:
        if m <= 32 and -(-n // 16) >= 4 * cus:
            nl = _stay_pieces(k, 1)
            if nl in (12, 16):
                return (-2, cus, nl), 1
        if narrow and m <= SKINNY_MAX_ROWS:
            parts = _fit_parts(-(-k // 256), min(4, cus // -(-n // 64)))
            if parts >= 2 and k >= parts * TILE64_MIN_SHARE:
                return TILE64, parts
            nl = _stay_pieces(k, 4)
            if nl is not None and -(-n // 16) * 2 <= PARTIAL_BLOCKS and (nl <= 5 or (m <= 32 and nl <= 8)):
                return (-2, cus, nl), 4
        return None
    tiles = -(-n // 16)
    if narrow and tiles <= PARTIAL_BLOCKS:
        for parts in (4, 2):                       # staying blocks: the more groups, the fewer registers hold x
            nl = _stay_pieces(k, parts)
            if nl is not None:
                # up to 8 pieces two blocks fit a compute unit, which pays up to an inner size of 4,096; beyond,
                # one block each walks its tiles (7,168 x 5,120 at 8 rows: 16.4 us against 16.9, and against
                # 18.9 with x resident in LDS; 5,120 x 8,192: 17.9 against 19.9 and 20.0)
                return (-2, (2 if nl <= 8 and k <= 4096 else 1) * cus, nl), parts
        parts = min(4, -(-PARTIAL_BLOCKS // tiles))
        parts = 4 if parts == 3 else parts
        if parts > 1:
            fewer = _fit_parts(-(-k // (PARTIAL_SHAPE[1] * PARTIAL_SHAPE[2] * 32)), parts)
            if fewer > 1 and not (m > 8 and n * k >= SKINNY_LARGE_MATRIX and k <= LIBRARY_MAX_INNER):
                return PARTIAL_SHAPE, fewer
    if tiles >= 4 * cus and (m >= 3 or tiles < 16 * cus):
        nl = _stay_pieces(k, 1)
        if nl is not None:
            return (-2, (2 if tiles >= 16 * cus else 1) * cus, nl), 1
    if m > 8 and n * k >= SKINNY_LARGE_MATRIX:
        return None
    return (0, 0, 0), 1


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype=None, partial_ok: bool = False, gate_pairs: "str | None" = None,
           partial_max_width: int | None = PARTIAL_SUM_MAX_WIDTH):
    """x @ w.T for w stored [out, in].

    float32: the library's own float-FMA kernel (no reduced-precision matrix mode).
    bfloat16, at most 16 rows (and some shapes up to 64): a weight-streaming MFMA kernel of this
    library (``streaming_plan``).
    bfloat16 otherwise: a plain library matrix product (hipBLASLt through torch), float accumulation.
    With ``partial_ok`` the caller takes a float32 stack [parts, M, N] of partial products as well
    (to be added in order, as ``add_rmsnorm`` does); it is returned for narrow matrices at up to 64 rows
    (``partial_max_width``: the widest row whose parts the caller's reader adds; None: any).
    With ``gate_pairs`` (one of ``GATE_ACTIVATIONS``) the rows of w alternate gate and up rows and the
    result is act(x.w[2j]) * (x.w[2j+1]) of width N/2 (an epilogue of the streaming kernels, a kernel
    of its own after the library's product).
    """
    scale = None
    if isinstance(x, UnscaledRows):
        scale, x = x, x.x
    if x.dtype == torch.float32:
        y = gemm_f32(x, w)
    else:
        _need(x.dtype == w.dtype, "x and w must have one type")
        plan = streaming_plan(x.shape[0], w.shape[0], w.shape[1], bool(gate_pairs),
                              partial_ok and out_dtype in (None, torch.bfloat16), x.device, partial_max_width)
        _need(scale is None or (plan is not None and plan[0][0] == -2),
              "un-normalised rows need a product by the blocks that stay (ask linear_takes_unscaled_rows first)")
        if plan is not None:
            shape, parts = plan
            if shape == TILE64:
                return gemm_tile64(x, w, torch.float32, ksplit=parts)
            if parts > 1:
                return gemm_skinny(x, w, torch.float32, block_shape=shape, ksplit=parts, row_scale=scale)
            return gemm_skinny(x, w, out_dtype or torch.bfloat16, gate_pairs=gate_pairs, block_shape=shape,
                               row_scale=scale)
        y = torch.mm(x, w.t())
    if gate_pairs:
        return gated_mul(y, interleaved=True, activation=gate_pairs)
    if out_dtype is not None and y.dtype != out_dtype:
        y = y.to(out_dtype)
    return y


def linear_takes_unscaled_rows(n_rows: int, w: torch.Tensor, gate_pairs: bool = False, partial_ok: bool = False,
                               partial_max_width: int | None = PARTIAL_SUM_MAX_WIDTH) -> bool:
    """Whether ``linear`` with these arguments multiplies ``UnscaledRows`` (its plan is the blocks that stay)."""
    if w.dtype != torch.bfloat16 or not unscaled_rows_possible(torch.bfloat16, n_rows, w.shape[1]):
        return False
    plan = streaming_plan(n_rows, w.shape[0], w.shape[1], bool(gate_pairs), partial_ok, w.device, partial_max_width)
    return plan is not None and plan[0] != TILE64 and plan[0][0] == -2


# --------------------------------------------------------------------------- sampling
def sample(logits: torch.Tensor, temperature=None, keys=None, out=None) -> torch.Tensor:
    """One token per row of float logits.  temperature[r] <= 0 (or None): greedy, lowest
    index among maxima; otherwise a draw from softmax(logits / temperature[r]) that depends
    on keys[r] (int64) and the row's logits only."""
    _dev(logits, temperature, keys)
    _f32(logits, "logits")
    m, v = logits.shape
    if temperature is not None:
        _f32(temperature, "temperature", m)
        _need(keys is not None and keys.dtype == torch.int64 and keys.numel() == m, "keys must be int64, one per row")
    if out is None:
        out = torch.empty((m,), dtype=torch.int32, device=logits.device)
    lib = library.core()
    lib.jv_sample_scratch_bytes.restype = c_longlong
    scratch = torch.empty(lib.jv_sample_scratch_bytes(c_int(m)), dtype=torch.uint8, device=logits.device)
    _check(lib.jv_sample(_ptr(out), _ptr(logits), c_longlong(v), c_int(m), c_int(v), _ptr(temperature),
                         _ptr(keys if temperature is not None else None), _ptr(scratch), _stream()), "sample")
    return out


# --------------------------------------------------------------------------- matrix-core attention (bfloat16)
MFMA_ATTENTION_MAX_HEAD_DIM = 256


def attn_prefill_geometry(head_dim: int) -> tuple[int, int]:
    """(rows of a group, groups a work item of the prefill kernel may name).  A row is a (query,
    head-in-group) pair."""
    return 64, (2 if head_dim <= 128 else 1)


def attn_prefill_waves_split(head_dim: int) -> bool:
    """Whether each group of a work item has waves of its own (head sizes 32, 64, 96, 128: two waves
    of 32 rows per group), so that a block is busy only while both groups see keys: neighbouring
    groups belong together.  Otherwise each of the 4 waves takes 16 rows of every group, and pairing
    a light group with a heavy one evens out the blocks."""
    return head_dim % 32 == 0 and head_dim <= 128


_checked_attention_libraries = set()


def _attention_library(head_dim: int):
    """The attention library of a head size; on its first use the numbers this module plans with
    (rows of a group, groups per work item, scratch size) are compared with the library's own."""
    lib = library.attention(head_dim)
    if head_dim not in _checked_attention_libraries:
        lib.jv_attn_decode_scratch_floats.restype = c_longlong
        got = (lib.jv_attn_head_dim(), lib.jv_attn_prefill_group_rows(), lib.jv_attn_prefill_groups_per_item(),
               bool(lib.jv_attn_prefill_waves_split()), lib.jv_attn_decode_scratch_floats(c_int(3), c_int(5), c_int(7)),
               lib.jv_attn_decode_table_entries(), lib.jv_attn_decode_tile_keys())
        want = (head_dim, *attn_prefill_geometry(head_dim), attn_prefill_waves_split(head_dim),
                attn_decode_scratch_floats(3, 5, 7, head_dim), ATTN_DECODE_TABLE_ENTRIES, ATTN_DECODE_TILE_KEYS)
        if got != want:
            raise KernelArgumentError(f"attention library for head size {head_dim} reports {got}, the planner expects {want}")
        _checked_attention_libraries.add(head_dim)
    return lib


def mfma_attention_supported(dtype, head_dim: int, page_size: int) -> bool:
    """The matrix-core kernels take bfloat16, head sizes that are multiples of 16 up to 256 and
    page sizes that are multiples of 8; everything else goes to the generic kernel."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= MFMA_ATTENTION_MAX_HEAD_DIM
            and page_size % 8 == 0)


def _attn_common(out, q, q_row_stride, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work, nq, nkv,
                 head_dim):
    _dev(out, q, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work)
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "matrix-core attention takes bfloat16")
    n = out.shape[0]
    _need(out.shape == (n, nq * head_dim), "out must be [tokens, nq * D]")
    _need(q_row_stride % 8 == 0 and q.data_ptr() % 16 == 0, "q rows must be 16-byte aligned")
    _need(q.numel() >= (n - 1) * q_row_stride + nq * head_dim if n else True, "q is too small for its stride")
    page_size = k_pages.shape[2]
    _check_pages(k_pages, v_pages, q.dtype, nkv, page_size, head_dim)
    _need(page_size % 8 == 0, "page size must be a multiple of 8")
    _need(block_tables.dim() == 2, "block_tables must be [requests, pages]")
    for t, name in ((block_tables, "block_tables"), (cu_seqlens, "cu_seqlens"), (context_lens, "context_lens"),
                    (work, "work")):
        if t is not None:
            _i32(t, name)
    _need(cu_seqlens.numel() == context_lens.numel() + 1 == block_tables.shape[0] + 1,
          "cu_seqlens, context_lens and block_tables disagree on the number of requests")
    return page_size


def _sinks_ok(sinks, nq: int) -> None:
    if sinks is not None:
        _dev(sinks)
        _f32(sinks, "sinks", nq)


def attn_prefill_mfma(out, q, q_row_stride, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work, n_work,
                      nq, nkv, head_dim, scale, window=0, sinks=None) -> None:
    """Causal attention of prompt portions.  ``work`` is int32 [n_work, 3]: (request index, first row
    of a group, first row of a second group of the same request or -1), see ``attn_prefill_geometry``;
    every row of every request must be in exactly one group.  Pairing a group that sees many keys with
    one that sees few gives all blocks the same amount of work.  ``sinks`` (float32 [nq]): exp(sinks[h]) joins every
    row's softmax denominator (a term without key and value, not scaled)."""
    _sinks_ok(sinks, nq)
    page_size = _attn_common(out, q, q_row_stride, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work,
                             nq, nkv, head_dim)
    _need(work.numel() >= 3 * n_work, "work list shorter than n_work")
    lib = _attention_library(head_dim)
    _check(
        lib.jv_attn_prefill(_ptr(out), _ptr(q), c_longlong(q_row_stride), _ptr(k_pages), _ptr(v_pages),
                            _ptr(block_tables), c_int(block_tables.shape[1]), _ptr(cu_seqlens), _ptr(context_lens),
                            _ptr(work), c_int(n_work), c_int(page_size), c_int(nq), c_int(nkv), c_float(scale),
                            c_int(window or 0), _ptr(sinks), _stream()),
        "attn_prefill_mfma",
    )


ATTN_DECODE_TABLE_ENTRIES = 4096    # page-table entries a block of the decode kernel keeps in LDS
ATTN_DECODE_TILE_KEYS = 32          # keys of one tile of the decode kernel


def attn_decode_min_splits(table_width: int, page_size: int) -> int:
    """The fewest splits with which the decode kernel takes block tables of this width: a row of up to
    4,096 entries is kept in LDS whole; of a wider one a block keeps the entries of its own split's
    keys, which must fit."""
    if table_width <= ATTN_DECODE_TABLE_ENTRIES:
        return 1
    tiles = -(-table_width * page_size // ATTN_DECODE_TILE_KEYS)
    tiles_per_split = (ATTN_DECODE_TABLE_ENTRIES - 2) * page_size // ATTN_DECODE_TILE_KEYS
    return -(-tiles // tiles_per_split)


def attn_decode_scratch_floats(n_work: int, nq: int, num_splits: int, head_dim: int) -> int:
    return n_work * nq * num_splits * (head_dim + 2) if num_splits > 1 else 0


def attn_decode_mfma(out, q, q_row_stride, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work, n_work,
                     nq, nkv, head_dim, scale, window=0, num_splits=1, scratch=None, sinks=None) -> None:
    """Attention of single decoded tokens.  ``work`` is int32 [n_work]: indices of the requests
    (each with exactly one token in this step); None: the step holds decoded tokens only, request
    r = 0 .. n_work-1 has its token in row r (the kernel then has nothing to look up before its
    loads start).  With ``num_splits`` > 1 a request's keys are shared out to that many blocks and
    ``scratch`` (float32, ``attn_decode_scratch_floats`` entries) holds their partial results.  ``sinks``: as for
    ``attn_prefill_mfma`` (counted once, after the splits are merged)."""
    _sinks_ok(sinks, nq)
    page_size = _attn_common(out, q, q_row_stride, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work,
                             nq, nkv, head_dim)
    if work is None:
        _need(n_work == context_lens.numel() == out.shape[0], "without a work list every request has one token")
    else:
        _need(work.numel() >= n_work, "work list shorter than n_work")
    _need(num_splits >= attn_decode_min_splits(block_tables.shape[1], page_size),
          f"block tables of {block_tables.shape[1]} pages need at least "
          f"{attn_decode_min_splits(block_tables.shape[1], page_size)} splits")
    if num_splits > 1:
        _need(scratch is not None and scratch.is_cuda and scratch.dtype == torch.float32
              and scratch.numel() >= attn_decode_scratch_floats(n_work, nq, num_splits, head_dim),
              "scratch too small for the splits")
    lib = _attention_library(head_dim)
    _check(
        lib.jv_attn_decode(_ptr(out), _ptr(q), c_longlong(q_row_stride), _ptr(k_pages), _ptr(v_pages),
                           _ptr(block_tables), c_int(block_tables.shape[1]),
                           _ptr(cu_seqlens if work is not None else None), _ptr(context_lens),
                           _ptr(work), c_int(n_work), c_int(page_size), c_int(nq), c_int(nkv), c_float(scale),
                           c_int(window or 0), c_int(num_splits), _ptr(scratch if num_splits > 1 else None),
                           _ptr(sinks), _stream()),
        "attn_decode_mfma",
    )


# --------------------------------------------------------------------------- what the chip delivers (for the measurement program)
def calibrate_read(buffer: torch.Tensor, sink: torch.Tensor, blocks: int = 2048) -> None:
    """Launch the kernel that only reads ``buffer`` (its byte size must split into 16-byte pieces
    evenly over ``blocks`` blocks); time it from outside."""
    _dev(buffer, sink)
    _f32(sink, "sink")
    n = buffer.numel() * buffer.element_size()
    _need(n % 16 == 0 and (n // 16) % blocks == 0, f"{n} bytes do not split into 16-byte pieces over {blocks} blocks")
    _check(library.core().jv_calibrate_read(_ptr(buffer), c_longlong(n), _ptr(sink), c_int(blocks), _stream()),
           "calibrate_read")


def calibrate_mfma(sink: torch.Tensor, turns: int, blocks: int) -> float:
    """Launch the kernel that only issues bf16 matrix-core products on registers; returns the
    floating-point operations it does."""
    _dev(sink)
    _f32(sink, "sink")
    lib = library.core()
    lib.jv_calibrate_mfma_flops.restype = ctypes.c_double
    _check(lib.jv_calibrate_mfma(_ptr(sink), c_int(turns), c_int(blocks), _stream()), "calibrate_mfma")
    return float(lib.jv_calibrate_mfma_flops(c_int(blocks), c_int(turns)))


# --------------------------------------------------------------------------- norms around a sublayer's output
class PendingNorm:
    """A sublayer's output ``y`` (rows of the activation type, or None) plus float partial results
    ``parts`` [P, rows, hidden] (or None) whose sum still has to be normed with ``weight`` before it
    joins the residual stream: what a layer arrangement that norms the output of its sublayers hands
    to the next norm, which does both in one pass (``postnorm_add_rmsnorm``)."""

    def __init__(self, y, parts, weight, eps: float, bias=None, scale: float = 1.0):
        self.y, self.parts, self.weight, self.eps = y, parts, weight, float(eps)
        self.bias = bias          # float [hidden] or None: a bias of the sublayer's last product, still to be added
        self.scale = float(scale)  # with ``weight`` None: no norm at all, the sum joins the stream times this constant


class BiasedOutput:
    """What a sublayer returned (rows, a float stack, or a pair of both) whose last product's bias [hidden] is
    still to be added: a block that norms the output lets the norm's kernel add it (``pending_norm``); anyone else
    calls ``settled()``."""

    def __init__(self, out, bias: torch.Tensor):
        self.out, self.bias = out, bias

    def settled(self):
        rows, parts = split_sublayer_output(self.out)
        add_bias(rows if rows is not None else parts, self.bias)
        return self.out


def split_sublayer_output(out):
    """(rows or None, float stack or None) of what a mixer or feed-forward returned: rows of the
    activation type, a float stack of partial results, or already a pair of both."""
    if isinstance(out, BiasedOutput):
        out = out.settled()
    if isinstance(out, tuple):
        return out
    if out.dim() == 3:
        return None, out
    return out, None


def pending_norm(out, weight: torch.Tensor, eps: float) -> "PendingNorm":
    """A sublayer's output with the norm that belongs to it, for the next norm's kernel; a bias that the output still
    owes travels along and is added there."""
    if isinstance(out, BiasedOutput):
        return PendingNorm(*split_sublayer_output(out.out), weight, eps, out.bias)
    return PendingNorm(*split_sublayer_output(out), weight, eps)


def pending_scale(out, scale: float) -> "PendingNorm":
    """A sublayer's output that joins the residual stream multiplied by a constant (no norm of its own): the next
    norm's kernel adds ``scale`` times the output (rows plus float partial results) and norms the stream in one pass."""
    if isinstance(out, BiasedOutput):
        out = out.settled()
    return PendingNorm(*split_sublayer_output(out), None, 0.0, None, scale)


def postnorm_add_rmsnorm(h, y, parts, post_weight, eps: float, weight=None, out=None, rows=None,
                         out_eps: float | None = None, bias=None, plain_scale: float = 1.0) -> None:
    """h += norm(y + parts[0] + parts[1] + ... (+ bias); post_weight) in the float residual stream, then, with
    ``out``, out = norm(h; weight) (with ``out_eps``, default ``eps``) in the activation type, or h itself in that type where
    ``weight`` is None (a reader that takes the stream as it is).  With ``rows`` (int32 indices) only those
    rows are computed and h is left alone.  ``post_weight`` None: the sublayer's output joins the stream under a constant
    only, h += plain_scale * (y + parts ...).  y is [rows of h, hidden] in the activation type or None,
    parts a float32 stack [P, rows of h, hidden] or None (any P)."""
    _dev(h, y, parts, post_weight, weight, out, rows, bias)
    _f32(h, "h")
    n, hidden = h.shape
    if post_weight is not None:
        _f32(post_weight, "post_weight", hidden)
    if bias is not None:       # added to the sublayer's output before its norm
        _f32(bias, "bias", hidden)
    _need(y is not None or parts is not None, "nothing to add")
    _need(hidden <= 16384, "rows wider than 16,384 are not supported")
    if y is not None:
        _need(y.shape == h.shape, "y must match h's shape")
    if parts is not None:
        _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[1:] == h.shape,
              "parts must be float32 [P, *h.shape]")
    if out is not None:
        if weight is not None:       # None: out is the stream itself in the activation type, not normed
            _f32(weight, "weight", hidden)
        n_out = out.shape[0]
        _need(out.shape[-1] == hidden, "out width differs from h")
        _need(y is None or y.dtype == out.dtype, "y and out must have one type")
    else:
        _need(rows is None, "rows without an output change nothing")
        n_out = n
    if rows is None:
        _need(n_out == n, "out must have one row per row of h")
    else:
        _i32(rows, "rows", n_out)
    kind = out.dtype if out is not None else (y.dtype if y is not None else torch.float32)
    fn = getattr(library.core(), f"jv_postnorm_add_rmsnorm_{_suffix(kind)}")
    _check(fn(_ptr(h), _ptr(y), _ptr(parts), c_int(0 if parts is None else parts.shape[0]),
              c_longlong(0 if parts is None else parts.stride(0)), _ptr(bias), _ptr(post_weight), _ptr(weight), _ptr(out),
              _ptr(rows), c_int(n_out), c_int(hidden), c_float(eps), c_float(eps if out_eps is None else out_eps), c_float(plain_scale), _stream()),
           "postnorm_add_rmsnorm")


def gated_rmsnorm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """norm(o; weight) * sigmoid(gate) for float rows ``o`` [n, width]; ``gate`` is a [n, width] view (unit
    column stride, any row stride) of the activation type, which is also the result's."""
    _dev(o, weight)
    _f32(o, "o")
    n, width = o.shape
    _f32(weight, "weight", width)
    _need(gate.is_cuda and gate.shape == o.shape and gate.stride(1) == 1, "gate must be a [n, width] view with unit column stride")
    out = torch.empty((n, width), dtype=gate.dtype, device=o.device)
    fn = getattr(library.core(), f"jv_gated_rmsnorm_{_suffix(gate.dtype)}")
    _check(fn(_ptr(out), _ptr(o), _ptr(gate), c_longlong(gate.stride(0)), _ptr(weight), c_int(n), c_int(width),
              c_float(eps), _stream()), "gated_rmsnorm")
    return out


# --------------------------------------------------------------------------- attention over a cached latent
def rope_table_amp(positions: torch.Tensor, inv_freq: torch.Tensor, amplitude: float) -> torch.Tensor:
    """``rope_table`` with cos and sin multiplied by a constant."""
    _dev(positions, inv_freq)
    n, half = positions.numel(), inv_freq.numel()
    _i32(positions, "positions")
    _f32(inv_freq, "inv_freq")
    out = torch.empty((n, 2 * half), dtype=torch.float32, device=positions.device)
    _check(library.core().jv_rope_table_amp(_ptr(out), _ptr(positions), _ptr(inv_freq), c_int(n), c_int(half),
                                            c_float(amplitude), _stream()), "rope_table_amp")
    return out


def latent_prepare(proj, q_rank: int, rank: int, rot: int, rot_dims: int, q_weight, kv_weight, eps: float, cos_sin,
                   slot_mapping, k_pages, v_pages, page_size: int, kv_off: "int | None" = None,
                   interleaved: bool = False):
    """From rows ``proj`` = [q latent | kv latent | key part to rotate | ...]: returns the normed q latent
    [n, q_rank] (None for ``q_rank`` 0: queries that are projected directly; the kv latent then begins at column
    ``kv_off``, default ``q_rank``); ``interleaved``: the pairs (2i, 2i + 1) turn instead of (i, i + rot_dims / 2); stores [normed kv latent | rotated key part] of every token with a slot (>= 0) into its key
    page [pages, 1, page_size, rank + rot] and transposed value page [pages, 1, rank + rot, page_size]."""
    _dev(proj, q_weight, kv_weight, cos_sin, slot_mapping, k_pages, v_pages)
    n, ld = proj.shape
    kv_off = q_rank if kv_off is None else int(kv_off)
    _need(q_rank >= 0 and kv_off >= q_rank and ld >= kv_off + rank + rot, "proj rows are too short")
    if q_rank:
        _f32(q_weight, "q_weight", q_rank)
    _f32(kv_weight, "kv_weight", rank)
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= rot, "the rotated size must be even and at most the key part")
    if rot_dims:
        _f32(cos_sin, "cos_sin", n * rot_dims)
    if k_pages is not None:
        _i32(slot_mapping, "slot_mapping", n)
        _check_pages(k_pages, v_pages, proj.dtype, 1, page_size, rank + rot)
    cq = torch.empty((n, q_rank), dtype=proj.dtype, device=proj.device) if q_rank else None
    fn = getattr(library.core(), f"jv_latent_prepare_{_suffix(proj.dtype)}")
    _check(fn(_ptr(proj), c_longlong(ld), c_int(n), c_int(q_rank), c_longlong(kv_off), c_int(rank), c_int(rot), c_int(rot_dims),
              c_int(1 if interleaved else 0), _ptr(q_weight if q_rank else None), _ptr(kv_weight), c_float(eps),
              _ptr(cos_sin if rot_dims else None),
              _ptr(slot_mapping if k_pages is not None else None), _ptr(cq), _ptr(k_pages), _ptr(v_pages),
              c_int(page_size), _stream()), "latent_prepare")
    return cq


def latent_query_rope(q, qe, heads: int, dim: int, rot: int, rot_dims: int, rank: int, cos_sin,
                      interleaved: bool = False) -> None:
    """qe[t, h, rank:] = rotate(q[t, h, dim:]) for q rows that begin with heads * (dim + rot) columns (further columns
    are left alone), qe [n, heads * (rank + rot)]; ``interleaved``: the pairs (2i, 2i + 1) turn."""
    _dev(q, qe, cos_sin)
    n = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] >= heads * (dim + rot) and qe.shape == (n, heads * (rank + rot)) and q.dtype == qe.dtype,
          "q rows must begin with heads * (dim + rot) columns, qe be [n, heads * (rank + rot)] of one type")
    if rot_dims:
        _f32(cos_sin, "cos_sin", n * rot_dims)
    fn = getattr(library.core(), f"jv_latent_query_rope_{_suffix(q.dtype)}")
    _check(fn(_ptr(q), c_longlong(q.shape[1]), _ptr(qe), c_int(n), c_int(heads), c_int(dim), c_int(rot), c_int(rot_dims),
              c_int(rank), _ptr(cos_sin if rot_dims else None), c_int(1 if interleaved else 0), _stream()), "latent_query_rope")


def head_linear(y, y_head_stride: int, x, x_head_stride: int, w, gate=None, matrix_cores: "bool | None" = None) -> None:
    """One matrix per head: y[t, h * ys : h * ys + N] = w[h] @ x[t, h * xs : h * xs + K], w [heads, N, K];
    with ``gate`` (a [n, heads * N] view with unit column stride) the result is multiplied by sigmoid(gate); a gate
    view [n, heads] holds one number per head, for all of the head's outputs.
    x and y are row-major matrices of the activation type; float accumulation.  bfloat16 with K, the row
    stride and the head stride of x multiples of 8 runs on the matrix cores (``matrix_cores`` False: the
    float-FMA kernels all the same)."""
    _dev(y, x, w)
    heads, N, K = w.shape
    n = x.shape[0]
    _need(x.dtype == w.dtype == y.dtype, "x, w and y must have one type")
    _need(y.shape[0] == n, "x and y differ in rows")
    _need((heads - 1) * x_head_stride + K <= x.shape[1] and (heads - 1) * y_head_stride + N <= y.shape[1],
          "heads do not fit the rows")
    if gate is not None:
        _need(gate.is_cuda and gate.dtype == x.dtype and gate.shape in ((n, heads * N), (n, heads)) and gate.stride(1) == 1,
              "gate must be a [n, heads * N] or [n, heads] view with unit column stride")
    possible = (x.dtype == torch.bfloat16 and K >= 8 and K % 8 == 0 and x.shape[1] % 8 == 0 and x_head_stride % 8 == 0
                and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
    _need(not matrix_cores or possible, "the matrix-core kernel takes bfloat16 and sizes and strides that are multiples of 8")
    name = "jv_head_linear_mfma_bf16" if possible and matrix_cores is not False else f"jv_head_linear_{_suffix(x.dtype)}"
    fn = getattr(library.core(), name)
    _check(fn(_ptr(y), c_longlong(y.shape[1]), c_int(y_head_stride), _ptr(x), c_longlong(x.shape[1]),
              c_int(x_head_stride), _ptr(w), c_int(n), c_int(N), c_int(K), c_int(heads), _ptr(gate),
              c_longlong(0 if gate is None else gate.stride(0)),
              c_int(N if gate is None or gate.shape[1] == heads * N else 1), _stream()), "head_linear")


# --------------------------------------------------------------------------- linear attention with decay
LIGHTNING_CHUNK_MIN_TOKENS = 8     # from this many tokens of a request on, the kernel by chunks


def lightning_max_dim(chunks: bool) -> int:
    return library.core().jv_lightning_max_dim(c_int(1 if chunks else 0))


def lightning_chunk_tokens() -> int:
    return library.core().jv_lightning_chunk_tokens()


def lightning_chunks_possible(dim: int) -> bool:
    """The kernels by chunks keep a chunk's keys in LDS in 16-byte pieces."""
    return dim % 4 == 0 and dim <= lightning_max_dim(True)


def lightning_chunk_plan(q_lens, device):
    """(work int32 [chunks, 2] = (request, first token row), first chunk of every request int32 [requests + 1],
    chunks) for the kernels by chunks: every request's tokens of this step cut into chunks, in order."""
    size = lightning_chunk_tokens()
    work, first, at = [], [0], 0
    for r, n in enumerate(q_lens):
        work += [(r, at + b) for b in range(0, n, size)]
        first.append(len(work))
        at += n
    flat = torch.tensor([x for w in work for x in w] + first, dtype=torch.int32).pin_memory().to(device, non_blocking=True)
    return flat[:2 * len(work)], flat[2 * len(work):], len(work)


def lightning_attention(proj, q_off: int, k_off: int, v_off: int, state, slot_ids, cu_seqlens, decay, heads: int,
                        dim: int, vdim: int, chunk_plan=None) -> torch.Tensor:
    """Float [n, heads * vdim]: o_t = S_t^T q_t with S_t = decay_h S_(t-1) + k_t v_t^T per request and head,
    q, k, v = silu of the columns of ``proj`` at the given offsets (head by head).  ``state``
    [slots + 1, heads, dim, vdim] float holds S of every request before the step and after it.
    ``chunk_plan`` (``lightning_chunk_plan`` of the step's token counts): the kernels that take a request's
    tokens a chunk at a time, chunks side by side, instead of one by one."""
    _dev(proj, state, slot_ids, cu_seqlens, decay)
    n, ld = proj.shape
    r = slot_ids.numel()
    _i32(slot_ids, "slot_ids")
    _i32(cu_seqlens, "cu_seqlens", r + 1)
    _f32(decay, "decay", heads)
    _f32(state, "state")
    _need(state.dim() == 4 and tuple(state.shape[1:]) == (heads, dim, vdim), "state must be [slots, heads, dim, vdim]")
    _need(max(q_off, k_off) + heads * dim <= ld and v_off + heads * vdim <= ld, "proj rows are too short")
    _need(dim <= lightning_max_dim(False), f"key size {dim} above the kernel's {lightning_max_dim(False)}")
    out = torch.empty((n, heads * vdim), dtype=torch.float32, device=proj.device)
    work = first = scratch = None
    chunks = 0
    if chunk_plan is not None:
        work, first, chunks = chunk_plan
        _need(lightning_chunks_possible(dim), "the kernels by chunks take key sizes that are multiples of 4, at most 128")
        _dev(work, first)
        _i32(work, "work", 2 * chunks)
        _i32(first, "first chunks", r + 1)
        scratch = torch.empty(chunks * heads * dim * vdim, dtype=torch.float32, device=proj.device)
    fn = getattr(library.core(), f"jv_lightning_{_suffix(proj.dtype)}")
    _check(fn(_ptr(out), _ptr(proj), c_longlong(ld), c_int(q_off), c_int(k_off), c_int(v_off), _ptr(state),
              _ptr(slot_ids), _ptr(cu_seqlens), _ptr(decay), c_int(r), c_int(heads), c_int(dim), c_int(vdim),
              c_int(chunks), _ptr(work), _ptr(first), _ptr(scratch), _stream()), "lightning_attention")
    return out


# --------------------------------------------------------------------------- recurrences with a matrix state
def short_conv_max_taps() -> int:
    return library.core().jv_short_conv_max_taps()


def recurrence_max_dim() -> int:
    return library.core().jv_recurrence_max_dim()


def short_conv(proj, c_off: int, channels: int, weight, bias, state, slot_ids, cu_seqlens, max_q_len: int,
               activation: bool = True) -> torch.Tensor:
    """Float [n, channels]: a causal convolution over time per channel of the columns ``proj[:, c_off : c_off +
    channels]``, request by request; ``weight`` [channels, taps] (the last column weighs the current token), ``bias``
    [channels] or None, then silu if ``activation``.  ``state`` [slots + 1, taps - 1, channels] float holds every
    request's last taps - 1 inputs before the step and after it (zeros stand before a sequence's first token)."""
    _dev(proj, weight, bias, state, slot_ids, cu_seqlens)
    n, ld = proj.shape
    r = slot_ids.numel()
    _need(weight.dim() == 2 and weight.shape[0] == channels, "weight must be [channels, taps]")
    taps = weight.shape[1]
    _f32(weight, "weight")
    _need(1 <= taps <= short_conv_max_taps(), f"a convolution of {taps} taps: the kernel takes up to {short_conv_max_taps()}")
    if bias is not None:
        _f32(bias, "bias", channels)
    _f32(state, "state")
    _need(state.dim() == 3 and tuple(state.shape[1:]) == (taps - 1, channels), "state must be [slots, taps - 1, channels]")
    _need(0 <= c_off and c_off + channels <= ld, "proj rows are too short")
    _i32(slot_ids, "slot_ids")
    _i32(cu_seqlens, "cu_seqlens", r + 1)
    out = torch.empty((n, channels), dtype=torch.float32, device=proj.device)
    fn = getattr(library.core(), f"jv_short_conv_{_suffix(proj.dtype)}")
    _check(fn(_ptr(out), c_longlong(channels), _ptr(proj), c_longlong(ld), c_int(c_off), c_int(channels), c_int(taps),
              _ptr(weight), _ptr(bias), _ptr(state), _ptr(slot_ids), _ptr(cu_seqlens), c_int(r), c_int(max(1, int(max_q_len))),
              c_int(1 if activation else 0), _stream()), "short_conv")
    return out


def recurrence_gates(proj, dt_off: int, dt_bias, a_log, heads: int, beta_off: "int | None" = None):
    """(decay, write strength), float [n, heads] each, from columns of ``proj``: dt = softplus(proj[:, dt_off + h] +
    dt_bias[h]) without a clamp, decay = exp(-exp(a_log[h]) * dt); the write strength is dt itself, or with
    ``beta_off`` sigmoid(proj[:, beta_off + h])."""
    _dev(proj, dt_bias, a_log)
    n, ld = proj.shape
    _f32(dt_bias, "dt_bias", heads)
    _f32(a_log, "a_log", heads)
    _need(0 <= dt_off and dt_off + heads <= ld and (beta_off is None or 0 <= beta_off and beta_off + heads <= ld), "proj rows are too short")
    g = torch.empty((n, heads), dtype=torch.float32, device=proj.device)
    w = torch.empty((n, heads), dtype=torch.float32, device=proj.device)
    fn = getattr(library.core(), f"jv_recurrence_gates_{_suffix(proj.dtype)}")
    _check(fn(_ptr(g), _ptr(w), _ptr(proj), c_longlong(ld), c_int(dt_off), c_int(0 if beta_off is None else beta_off),
              _ptr(dt_bias), _ptr(a_log), c_int(n), c_int(heads), c_int(0 if beta_off is None else 1), _stream()), "recurrence_gates")
    return g, w


def heads_to_f32(proj, off: int, heads: int, d: int, rot_dims: int = 0, cos_sin=None, scale: float = 1.0) -> torch.Tensor:
    """Float [n, heads * d] of the columns ``proj[:, off : off + heads * d]``; the first ``rot_dims`` elements of every
    head turn by the token's angles (``rope_table``; element i pairs with i + rot_dims / 2); all times ``scale``."""
    _dev(proj, cos_sin)
    n, ld = proj.shape
    _need(0 <= off and off + heads * d <= ld, "proj rows are too short")
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= d, "the rotated size must be even and at most the head size")
    if rot_dims:
        _f32(cos_sin, "cos_sin", n * rot_dims)
    out = torch.empty((n, heads * d), dtype=torch.float32, device=proj.device)
    fn = getattr(library.core(), f"jv_heads_to_f32_{_suffix(proj.dtype)}")
    _check(fn(_ptr(out), _ptr(proj), c_longlong(ld), c_int(off), c_int(n), c_int(heads), c_int(d), c_int(rot_dims),
              _ptr(cos_sin if rot_dims else None), c_float(scale), _stream()), "heads_to_f32")
    return out


def qkv_to_f32(proj, heads: int, d: int, dv: int, rot_dims: int = 0, cos_sin=None, k_scale: float = 1.0) -> torch.Tensor:
    """Float [n, 2 * heads * d + heads * dv] = [q | k | v] of the leading columns of ``proj`` laid out the same way: the
    first ``rot_dims`` elements of every q and k head turn by the token's angles (``rope_table``), k is multiplied by
    ``k_scale``, v is copied: ``heads_to_f32`` for the three inputs of one mixer in one launch."""
    _dev(proj, cos_sin)
    n, ld = proj.shape
    width = 2 * heads * d + heads * dv
    _need(width <= ld, "proj rows are too short")
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= d, "the rotated size must be even and at most the head size")
    if rot_dims:
        _f32(cos_sin, "cos_sin", n * rot_dims)
    out = torch.empty((n, width), dtype=torch.float32, device=proj.device)
    fn = getattr(library.core(), f"jv_qkv_to_f32_{_suffix(proj.dtype)}")
    _check(fn(_ptr(out), _ptr(proj), c_longlong(ld), c_int(n), c_int(heads), c_int(d), c_int(dv), c_int(rot_dims),
              _ptr(cos_sin if rot_dims else None), c_float(k_scale), _stream()), "qkv_to_f32")
    return out


def head_unit_norm(x: torch.Tensor, heads: int, d: int, eps: float, scale: float = 1.0, first_heads: int = 0,
                   first_scale: float = 1.0) -> None:
    """In place on float rows [n, width]: each of the first ``heads`` runs of ``d`` columns of every row becomes
    x / sqrt(sum(x^2) + eps) * scale; the first ``first_heads`` of them take ``first_scale`` instead."""
    _dev(x)
    _f32(x, "x")
    _need(x.dim() == 2 and d > 0 and heads * d <= x.shape[1], "the heads do not fit the rows")
    _check(library.core().jv_head_unit_norm(_ptr(x), c_longlong(x.shape[1]), c_longlong(x.shape[0]), c_int(heads), c_int(d),
                                            c_float(eps), c_int(first_heads), c_float(first_scale), c_float(scale), _stream()),
           "head_unit_norm")


def recurrence_steps(q, k, v, decay, state, slot_ids, cu_seqlens, heads: int, qk_heads: int, dim: int, vdim: int,
                     write=None, skip=None, delta: bool = False, chunk_plan=None) -> torch.Tensor:
    """Float [n, heads * vdim], token by token per request and head, S [dim, vdim] float in the request's state row:

        S <- g S;   u = w (v - S^T k) if ``delta`` else w v;   S <- S + k u^T;   o = S^T q + skip[h] v

    ``q``, ``k``: float views [n, qk_heads * dim] (unit column stride; head h reads q/k head h // (heads // qk_heads)),
    ``v`` a float view [n, heads * vdim]; ``decay`` g: float [n, heads] or [heads] (constant per head); ``write`` w:
    float [n, heads] or None (1); ``skip``: float [heads] or None.  ``chunk_plan`` (``recurrence_chunk_plan`` of the
    step's token counts): the kernels that take a request's tokens a chunk at a time, chunks side
    by side, instead of one by one (the same numbers in another order of operations)."""
    _dev(decay, write, skip, state, slot_ids, cu_seqlens)
    n = v.shape[0]
    r = slot_ids.numel()
    for name, t, width in (("q", q, qk_heads * dim), ("k", k, qk_heads * dim), ("v", v, heads * vdim)):
        _need(t.is_cuda and t.dtype == torch.float32 and t.dim() == 2 and t.shape == (n, width) and (n == 0 or t.stride(1) == 1),
              f"{name} must be a float [n, {width}] view with unit column stride")
    _need(heads % qk_heads == 0, "heads must be a multiple of the q/k heads")
    _f32(decay, "decay")
    _need(tuple(decay.shape) in ((n, heads), (heads,)), "decay must be [n, heads] or [heads]")
    if write is not None:
        _f32(write, "write", n * heads)
    if skip is not None:
        _f32(skip, "skip", heads)
    _f32(state, "state")
    _need(state.dim() == 4 and tuple(state.shape[1:]) == (heads, dim, vdim), "state must be [slots, heads, dim, vdim]")
    _need(dim <= recurrence_max_dim(), f"key size {dim} above the kernel's {recurrence_max_dim()}")
    _i32(slot_ids, "slot_ids")
    _i32(cu_seqlens, "cu_seqlens", r + 1)
    out = torch.empty((n, heads * vdim), dtype=torch.float32, device=v.device)
    if n == 0:
        return out
    if chunk_plan is not None:
        work, first, chunks = chunk_plan
        _need(recurrence_chunks_possible(dim, delta), "the kernels by chunks take key sizes that are multiples of 4, at most 128")
        _dev(work, first)
        _i32(work, "work", 2 * chunks)
        _i32(first, "first chunks", r + 1)
        cum = torch.empty(n * heads, dtype=torch.float32, device=v.device)
        if delta:
            _need(skip is None, "the delta rule by chunks has no skip term")
            lib = library.core()
            lib.jv_delta_chunks_scratch_floats.restype = c_longlong
            scratch = torch.empty(lib.jv_delta_chunks_scratch_floats(c_int(chunks), c_int(n), c_int(heads), c_int(dim), c_int(vdim)),
                                  dtype=torch.float32, device=v.device)
            _check(lib.jv_delta_chunks(
                _ptr(out), _ptr(q), c_longlong(q.stride(0)), _ptr(k), c_longlong(k.stride(0)), _ptr(v), c_longlong(v.stride(0)),
                _ptr(decay), c_int(heads if decay.dim() == 2 else 0), _ptr(write), _ptr(state), _ptr(slot_ids), _ptr(cu_seqlens),
                c_int(r), c_int(n), c_int(heads), c_int(qk_heads), c_int(dim), c_int(vdim), c_int(chunks), _ptr(work), _ptr(first),
                _ptr(scratch), _ptr(cum), _stream()), "delta_chunks")
            return out
        scratch = torch.empty(chunks * heads * dim * vdim, dtype=torch.float32, device=v.device)
        _check(library.core().jv_recurrence_chunks(
            _ptr(out), _ptr(q), c_longlong(q.stride(0)), _ptr(k), c_longlong(k.stride(0)), _ptr(v), c_longlong(v.stride(0)),
            _ptr(decay), c_int(heads if decay.dim() == 2 else 0), _ptr(write), _ptr(skip), _ptr(state), _ptr(slot_ids),
            _ptr(cu_seqlens), c_int(r), c_int(heads), c_int(qk_heads), c_int(dim), c_int(vdim), c_int(chunks), _ptr(work),
            _ptr(first), _ptr(scratch), _ptr(cum), _stream()), "recurrence_chunks")
        return out
    _check(library.core().jv_recurrence_steps(
        _ptr(out), _ptr(q), c_longlong(q.stride(0)), _ptr(k), c_longlong(k.stride(0)), _ptr(v), c_longlong(v.stride(0)),
        _ptr(decay), c_int(heads if decay.dim() == 2 else 0), _ptr(write), _ptr(skip), _ptr(state), _ptr(slot_ids),
        _ptr(cu_seqlens), c_int(r), c_int(heads), c_int(qk_heads), c_int(dim), c_int(vdim), c_int(1 if delta else 0), _stream()),
        "recurrence_steps")
    return out


def token_shift_mix(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, slot_ids, cu_seqlens, token_req) -> torch.Tensor:
    """Blends of every row with the row before it in its request: returns [S, n, hidden] of x's type with
    out[s, t] = x[t] + (x[t-1] - x[t]) * mu[s] (float arithmetic); ``mu`` float32 [S, hidden].  The row before a
    request's first row of the step is the request's row of ``state`` (float32 [slots + 1, hidden], zeros for a
    request that starts), which then takes the request's last row of the step."""
    _dev(x, mu, state, slot_ids, cu_seqlens, token_req)
    n, hidden = x.shape
    _f32(mu, "mu")
    _need(mu.dim() == 2 and mu.shape[1] == hidden, "mu must be [S, hidden]")
    _f32(state, "state")
    _need(state.dim() == 2 and state.shape[1] == hidden, "the state must be [slots + 1, hidden]")
    _i32(slot_ids, "slot_ids")
    _i32(cu_seqlens, "cu_seqlens", slot_ids.numel() + 1)
    _i32(token_req, "token_req", n)
    out = torch.empty((mu.shape[0], n, hidden), dtype=x.dtype, device=x.device)
    fn = getattr(library.core(), f"jv_token_shift_mix_{_suffix(x.dtype)}")
    _check(fn(_ptr(out), _ptr(x), _ptr(mu), c_int(mu.shape[0]), _ptr(state), _ptr(slot_ids), _ptr(cu_seqlens), _ptr(token_req),
              c_longlong(n), c_int(hidden), _stream()), "token_shift_mix")
    return out


WKV_MAX_DIM = 8192      # 32 rows of a column in each of a block's 256 threads


WKV_CHUNK_MIN_TOKENS = 8      # from this many tokens of a request on, the kernels by chunks
WKV_CHUNK_MAX_DIM = 128       # key channels of a head whose chunk fits a block's LDS
WKV_CHUNK_TOKENS = 32


def wkv_chunk_plan(ctx, dim: int):
    """The chunk plan of a step for ``wkv_steps`` (work int32 [chunks, 2] = (request, first token row), first chunk of
    every request int32 [requests + 1], chunks), or None where the step runs token by token: a recorded step, a step of
    short portions only, heads wider than the kernels by chunks take.  One plan serves every such layer of the step."""
    if ctx.captured or ctx.max_q_len < WKV_CHUNK_MIN_TOKENS or dim > WKV_CHUNK_MAX_DIM:
        return None
    plan = ctx.plans.get("wkv_chunks")
    if plan is None:
        _need(int(library.core().jv_wkv_chunk_tokens()) == WKV_CHUNK_TOKENS, "the library's chunks have another size")
        work, first, at = [], [0], 0
        for r, n in enumerate(ctx.q_lens_host):
            work += [(r, at + b) for b in range(0, n, WKV_CHUNK_TOKENS)]
            first.append(len(work))
            at += n
        flat = torch.tensor([x for w in work for x in w] + first, dtype=torch.int32).pin_memory().to(ctx.positions.device, non_blocking=True)
        plan = ctx.plans["wkv_chunks"] = (flat[:2 * len(work)], flat[2 * len(work):], len(work))
    return plan


def wkv_steps(r, k, v, rate, w0, bonus, state, slot_ids, cu_seqlens, heads: int, dim: int, vdim: int,
              chunk_plan=None) -> torch.Tensor:
    """The recurrence with a decay per key channel and a bonus for the current token, per head with S the request's
    float state [dim, vdim]:  w = exp(-exp(rate + w0));  o = S^T r + (sum_d r[d] bonus[d] k[d]) v;  S <- diag(w) S + k v^T.
    r, k, rate [n, heads * dim] and v [n, heads * vdim] are views (unit column stride) of the activation type; w0 and
    bonus float32 [heads * dim]; ``state`` float32 [slots + 1, heads, dim, vdim].  Returns float32 [n, heads * vdim].
    With ``chunk_plan`` (``wkv_chunk_plan``) the chunks of every request run side by side and only the states between
    them are walked in order; the results differ from the token-by-token kernel's by rounding."""
    _dev(w0, bonus, state, slot_ids, cu_seqlens)
    n = r.shape[0]
    for name, t, width in (("r", r, heads * dim), ("k", k, heads * dim), ("rate", rate, heads * dim), ("v", v, heads * vdim)):
        _need(t.is_cuda and t.dtype == r.dtype and t.shape == (n, width) and (n == 0 or t.stride(1) == 1),
              f"{name} must be a [n, {width}] view with unit column stride of one type")
    _f32(w0, "w0", heads * dim)
    _f32(bonus, "bonus", heads * dim)
    _f32(state, "state")
    _need(state.dim() == 4 and tuple(state.shape[1:]) == (heads, dim, vdim), "the state must be [slots + 1, heads, dim, vdim]")
    _i32(slot_ids, "slot_ids")
    _i32(cu_seqlens, "cu_seqlens", slot_ids.numel() + 1)
    out = torch.empty((n, heads * vdim), dtype=torch.float32, device=r.device)
    if chunk_plan is not None:
        work, req_chunks, chunks = chunk_plan
        _need(dim <= WKV_CHUNK_MAX_DIM, "heads too wide for the kernels by chunks")
        _i32(work, "work", 2 * chunks)
        _i32(req_chunks, "req_chunks", slot_ids.numel() + 1)
        floats = torch.empty(chunks * heads * dim * vdim + n * heads * dim + chunks * heads * dim, dtype=torch.float32,
                             device=r.device)
        scratch = floats[:chunks * heads * dim * vdim]
        rq = floats[scratch.numel():scratch.numel() + n * heads * dim]
        dtot = floats[scratch.numel() + rq.numel():]
        fn = getattr(library.core(), f"jv_wkv_chunks_{_suffix(r.dtype)}")
        _check(fn(_ptr(out), _ptr(r), c_longlong(r.stride(0)), _ptr(k), c_longlong(k.stride(0)), _ptr(v), c_longlong(v.stride(0)),
                  _ptr(rate), c_longlong(rate.stride(0)), _ptr(w0), _ptr(bonus), _ptr(state), _ptr(slot_ids), _ptr(cu_seqlens),
                  c_int(slot_ids.numel()), c_int(heads), c_int(dim), c_int(vdim), c_int(chunks), _ptr(work), _ptr(req_chunks),
                  _ptr(scratch), _ptr(rq), _ptr(dtot), _stream()), "wkv_chunks")
        return out
    fn = getattr(library.core(), f"jv_wkv_steps_{_suffix(r.dtype)}")
    _check(fn(_ptr(out), _ptr(r), c_longlong(r.stride(0)), _ptr(k), c_longlong(k.stride(0)), _ptr(v), c_longlong(v.stride(0)),
              _ptr(rate), c_longlong(rate.stride(0)), _ptr(w0), _ptr(bonus), _ptr(state), _ptr(slot_ids), _ptr(cu_seqlens),
              c_int(slot_ids.numel()), c_int(heads), c_int(dim), c_int(vdim), _stream()), "wkv_steps")
    return out


RECURRENCE_CHUNK_MIN_TOKENS = 8     # from this many tokens of a request on, the kernels by chunks


def recurrence_chunk_tokens() -> int:
    return library.core().jv_recurrence_chunk_tokens()


def recurrence_chunks_possible(dim: int, delta: bool = False) -> bool:
    """The kernels by chunks (of the plain recurrence and of the delta rule alike) keep a chunk's keys in LDS in
    16-byte pieces."""
    return dim % 4 == 0 and dim <= library.core().jv_recurrence_chunk_max_dim()


def recurrence_chunk_plan(q_lens, device):
    """(work int32 [chunks, 2] = (request, first token row), first chunk of every request int32 [requests + 1],
    chunks) for the recurrence by chunks: every request's tokens of this step cut into chunks, in order."""
    size = recurrence_chunk_tokens()
    work, first, at = [], [0], 0
    for r, n in enumerate(q_lens):
        work += [(r, at + b) for b in range(0, n, size)]
        first.append(len(work))
        at += n
    flat = torch.tensor([x for w in work for x in w] + first, dtype=torch.int32).pin_memory().to(device, non_blocking=True)
    return flat[:2 * len(work)], flat[2 * len(work):], len(work)


def step_chunk_plan(ctx, dim: int, delta: bool = False):
    """The chunk plan of a step for a recurrence with keys of ``dim`` elements, or None where the step runs token by
    token: a recorded step, a step of short portions only, sizes the kernels by chunks are not built for.  One plan
    serves every such layer of the step (``ctx.plans``)."""
    if ctx.captured or ctx.max_q_len < RECURRENCE_CHUNK_MIN_TOKENS or not recurrence_chunks_possible(dim, delta):
        return None
    plan = ctx.plans.get("recurrence_chunks")
    if plan is None:
        plan = ctx.plans["recurrence_chunks"] = recurrence_chunk_plan(ctx.q_lens_host, ctx.positions.device)
    return plan


NORM_GATES = {"silu": 1, "sigmoid": 2}


def group_gated_norm(o: torch.Tensor, gate: torch.Tensor, weight, group: int, eps: float, gate_activation: str = "silu",
                     gate_first: bool = False, out_scale: float = 1.0) -> torch.Tensor:
    """Float rows ``o`` [n, width] normed in equal groups of ``group`` columns (each by its own root mean square), times
    ``weight`` (float, any length that divides the width: it repeats; None: no weight), with act(gate) multiplied in
    before the norm (``gate_first``) or behind it, times ``out_scale``; ``gate`` is a [n, width] view (unit column
    stride) of the activation type, which is also the result's."""
    _dev(o, weight)
    _f32(o, "o")
    n, width = o.shape
    _need(group > 0 and width % group == 0, "the width must be whole groups")
    _need(gate_activation in NORM_GATES, f"gate activation {gate_activation!r}: one of {sorted(NORM_GATES)}")
    period = 0
    if weight is not None:
        _f32(weight, "weight")
        period = weight.numel()
        _need(period > 0 and width % period == 0, "the weight's length must divide the width")
    _need(gate.is_cuda and gate.shape == o.shape and (n == 0 or gate.stride(1) == 1), "gate must be a [n, width] view with unit column stride")
    out = torch.empty((n, width), dtype=gate.dtype, device=o.device)
    fn = getattr(library.core(), f"jv_group_gated_norm_{_suffix(gate.dtype)}")
    _check(fn(_ptr(out), _ptr(o), _ptr(gate), c_longlong(gate.stride(0) if n else 0), _ptr(weight), c_int(period), c_int(n),
              c_int(width), c_int(group), c_float(eps), c_int(NORM_GATES[gate_activation]), c_int(1 if gate_first else 0),
              c_float(out_scale), _stream()), "group_gated_norm")
    return out


# --------------------------------------------------------------------------- routed experts
def moe_tile_rows() -> int:
    """Rows of a tile of the float-FMA expert kernels (the matrix-core ones also take tiles of 128)."""
    return library.core().jv_moe_tile_rows()


def moe_tile_rows_for(dtype, hidden: int, ff: int, entries: int, experts: int) -> int:
    """Rows of a tile for a step: 128 where the matrix-core kernels run and an expert gets about a
    hundred rows or more (a row of W then feeds twice the products), else 64."""
    if moe_matrix_cores_possible(dtype, hidden, ff) and entries >= 96 * experts:
        return 128
    return moe_tile_rows()


ROUTER_FUSED_MAX_ROWS = 64      # 17..64 rows: logits and choice in one launch


def gemm_rows_f32out(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """float32 x @ w.T for bfloat16 x [M, K] and w [N, K] on the matrix cores (K a multiple of 8): products
    whose result must not be rounded to the activation type (router logits)."""
    _dev(x, w)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_rows_f32out takes bfloat16")
    m, k = x.shape
    n = w.shape[0]
    _need(w.shape[1] == k and k % 8 == 0 and k >= 8, "inner sizes must agree and be a multiple of 8")
    out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _check(library.core().jv_gemm_rows_f32out_bf16(_ptr(out), _ptr(x), _ptr(w), c_int(m), c_int(n), c_int(k), _stream()),
           "gemm_rows_f32out")
    return out


class MoePlan:
    """Device-side grouping of a step's (token, choice) entries by expert."""

    def __init__(self, ids, weights, meta, offsets, tile_expert, tile_row0, order, max_tiles, top, tile_rows):
        self.ids, self.weights, self.meta, self.offsets = ids, weights, meta, offsets
        self.tile_expert, self.tile_row0, self.order, self.max_tiles, self.top = tile_expert, tile_row0, order, max_tiles, top
        self.tile_rows = tile_rows


ROUTER_SCORES = {"sigmoid": 0, "softmax_chosen": 1, "sigmoid_normed": 2}      # the kernels' ids of how a chosen logit becomes a weight


def moe_route(logits: "torch.Tensor | None", top: int, x=None, w_router=None, logits_out=None,
              tile_rows: "int | None" = None, bias=None, score: str = "sigmoid", correction=None,
              weight_scale: float = 1.0) -> MoePlan:
    """Chooses for every token the ``top`` experts with the largest router logits (the lowest index among equal
    logits) and orders the n * top entries by expert, all on the device.  ``bias`` (float32 [experts]) is added
    to the logits before the choice; ``score``: a chosen expert's weight is "sigmoid" of its logit, or
    "softmax_chosen": the softmax over the token's chosen logits alone, or "sigmoid_normed": the experts with the
    largest sigmoid(logit) + ``correction`` (float32 [experts] or None) are chosen, and a chosen expert's weight is its
    sigmoid(logit) (without the correction) over the sum of the chosen ones' (+ 1e-20), times ``weight_scale``.
    Either float ``logits`` [n, experts] are given, or rows ``x`` [n, hidden] and the router matrix
    ``w_router`` [experts, hidden] of one type: then the logits are made here, in float (``logits_out``,
    float32 [n, experts], receives them if given): in the same launch as the choice (float32, odd sizes), or
    for bfloat16 by a matrix-core product with float output before it.  ``tile_rows``: rows of a tile of the grouping
    (``moe_tile_rows_for``; default: the float-FMA kernels' 64)."""
    if (logits is None and x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and x.shape[1] >= 8
            and w_router.shape[0] <= 3840):
        # bfloat16: the logits come from a matrix-core product with float output (never rounded to bfloat16): the
        # weight-streaming one for the few rows of a decode step, the tiled one for prompt portions; between
        # them (measured at 32 rows: one block of the tiled product walks the whole router alone) the fused kernel
        rows = x.shape[0]
        plan = streaming_plan(rows, w_router.shape[0], w_router.shape[1], device=x.device) if rows <= SKINNY_AUTO_ROWS else None
        if plan is not None and plan[1] == 1:
            logits = gemm_skinny(x, w_router, torch.float32, block_shape=plan[0])
        elif rows > ROUTER_FUSED_MAX_ROWS:
            logits = gemm_rows_f32out(x, w_router)
        if logits is not None and logits_out is not None:
            logits_out.copy_(logits if bias is None else logits + bias)
    _need(score in ROUTER_SCORES, f"no router score {score!r}: there are {sorted(ROUTER_SCORES)}")
    if logits is not None:
        _dev(logits)
        _f32(logits, "logits")
        n, experts = logits.shape
        dev = logits.device
    else:
        _dev(x, w_router, logits_out)
        n, hidden = x.shape
        experts = w_router.shape[0]
        _need(w_router.shape == (experts, hidden) and w_router.dtype == x.dtype, "the router must be [experts, hidden] of x's type")
        _need(hidden + experts <= 15000, "row and router too wide for the router kernel")
        if logits_out is not None:
            _f32(logits_out, "logits_out", n * experts)
        dev = x.device
    _need(0 < top <= experts, "top must be between 1 and the number of experts")
    if bias is not None:
        _dev(bias)
        _f32(bias, "bias", experts)
    _need(score == "sigmoid_normed" or (correction is None and weight_scale == 1.0),
          "a correction of the choice and a constant on the weights belong to the score 'sigmoid_normed'")
    if correction is not None:
        _dev(correction)
        _f32(correction, "correction", experts)
    entries = n * top
    tile_rows = tile_rows or moe_tile_rows()
    _need(tile_rows in (64, 128), "tiles have 64 or 128 rows")
    max_tiles = -(-entries // tile_rows) + experts
    ints = torch.empty(entries * 3 + 1 + experts + 1 + 2 * max_tiles, dtype=torch.int32, device=dev)
    ids, rank, order = ints[:entries], ints[entries:2 * entries], ints[2 * entries:3 * entries]
    at = 3 * entries
    meta, offsets = ints[at:at + 1], ints[at + 1:at + 2 + experts]
    at += 2 + experts
    tile_expert, tile_row0 = ints[at:at + max_tiles], ints[at + max_tiles:at + 2 * max_tiles]
    weights = torch.empty(entries, dtype=torch.float32, device=dev)
    lib = library.core()
    if logits is not None:
        _check(lib.jv_moe_route(_ptr(logits), _ptr(bias), c_int(n), c_int(experts), c_int(top), c_int(ROUTER_SCORES[score]),
                                _ptr(ids), _ptr(weights), _ptr(correction), c_float(weight_scale), _stream()), "moe_route")
    else:
        _check(getattr(lib, f"jv_moe_router_{_suffix(x.dtype)}")(
            _ptr(x), _ptr(w_router), _ptr(bias), c_int(n), c_int(hidden), c_int(experts), c_int(top),
            c_int(ROUTER_SCORES[score]), _ptr(ids), _ptr(weights), _ptr(logits_out), _ptr(correction),
            c_float(weight_scale), _stream()), "moe_router")
    _check(lib.jv_moe_group(_ptr(ids), c_int(entries), c_int(experts), c_int(tile_rows), _ptr(meta), _ptr(offsets), _ptr(tile_expert),
                            _ptr(tile_row0), _ptr(order), _ptr(rank), _stream()), "moe_group")
    return MoePlan(ids, weights, meta, offsets, tile_expert, tile_row0, order, max_tiles, top, tile_rows)


def row_gate(out: torch.Tensor, y: torch.Tensor, gate: torch.Tensor) -> None:
    """out[t] = float(y[t]) * sigmoid(gate[t]): rows ``y`` [n, hidden] of the activation type under one gate per row
    (``gate`` a [n, 1] view of the same type, any row stride), into float32 ``out`` [n, hidden]."""
    _dev(out, y)
    n, hidden = y.shape
    _need(out.dtype == torch.float32 and out.shape == y.shape, "out must be float32 of y's shape")
    _need(gate.is_cuda and gate.dtype == y.dtype and gate.shape == (n, 1), "gate must be a [n, 1] view of y's type")
    fn = getattr(library.core(), f"jv_row_gate_{_suffix(y.dtype)}")
    _check(fn(_ptr(out), _ptr(y), _ptr(gate), c_longlong(gate.stride(0)), c_longlong(n), c_int(hidden), _stream()), "row_gate")


def moe_matrix_cores_possible(dtype, hidden: int, ff: int) -> bool:
    """The grouped products have a matrix-core form for bfloat16 and inner sizes that are multiples of 8."""
    return dtype == torch.bfloat16 and hidden % 8 == 0 and ff % 8 == 0 and hidden >= 8 and ff >= 8


def moe_experts(x, plan: MoePlan, w_gate, w_up, w_down, activation: str, out: torch.Tensor,
                weight_on_input: bool = True, matrix_cores: "bool | None" = None) -> None:
    """out[kk, t] = down[e] (act(gate[e] xs) * (up[e] xs)) for the kk-th chosen expert e of token t, float32
    [top, n, hidden]; xs = weight * x[t] with ``weight_on_input``, else x[t] and the result is multiplied
    by the weight.  w_gate, w_up [experts, ff, hidden], w_down [experts, hidden, ff].  ``matrix_cores``:
    None takes the matrix-core kernels wherever ``moe_matrix_cores_possible``, False the float-FMA ones."""
    _dev(x, w_gate, w_up, w_down, out)
    n, hidden = x.shape
    experts, ff, _ = w_gate.shape
    _need(w_gate.shape == w_up.shape == (experts, ff, hidden) and w_down.shape == (experts, hidden, ff),
          "expert weights must be [experts, ff, hidden] and [experts, hidden, ff]")
    _need(x.dtype == w_gate.dtype == w_up.dtype == w_down.dtype, "x and the weights must have one type")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (plan.top, n, hidden), "out must be float32 [top, n, hidden]")
    _need(plan.ids.numel() == n * plan.top, "the plan belongs to another step")
    z = torch.empty((n * plan.top, ff), dtype=x.dtype, device=x.device)
    lib, suf = library.core(), _suffix(x.dtype)
    possible = moe_matrix_cores_possible(x.dtype, hidden, ff)
    _need(not matrix_cores or possible, "the matrix-core kernels take bfloat16 and inner sizes that are multiples of 8")
    mfma = possible and matrix_cores is not False
    _need(mfma or plan.tile_rows == moe_tile_rows(), "the float-FMA kernels take tiles of 64 rows")
    p = plan
    if mfma:
        _check(lib.jv_moe_gate_up_mfma_bf16(
            _ptr(z), _ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(p.meta), _ptr(p.offsets), _ptr(p.tile_expert),
            _ptr(p.tile_row0), _ptr(p.order), _ptr(p.weights), c_int(p.max_tiles), c_int(p.top), c_int(hidden), c_int(ff),
            c_int(_gate_act_id(activation)), c_int(1 if weight_on_input else 0), c_int(p.tile_rows), _stream()), "moe_gate_up")
        _check(lib.jv_moe_down_mfma_bf16(
            _ptr(out), _ptr(z), _ptr(w_down), _ptr(p.meta), _ptr(p.offsets), _ptr(p.tile_expert), _ptr(p.tile_row0),
            _ptr(p.order), _ptr(p.weights), c_int(p.max_tiles), c_int(p.top), c_int(n), c_int(hidden), c_int(ff),
            c_int(0 if weight_on_input else 1), c_int(p.tile_rows), _stream()), "moe_down")
        return
    _check(getattr(lib, f"jv_moe_gate_up_{suf}")(
        _ptr(z), _ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(p.meta), _ptr(p.offsets), _ptr(p.tile_expert),
        _ptr(p.tile_row0), _ptr(p.order), _ptr(p.weights), c_int(p.max_tiles), c_int(p.top), c_int(hidden), c_int(ff),
        c_int(_gate_act_id(activation)), c_int(1 if weight_on_input else 0), _stream()), "moe_gate_up")
    _check(getattr(lib, f"jv_moe_down_{suf}")(
        _ptr(out), _ptr(z), _ptr(w_down), _ptr(p.meta), _ptr(p.offsets), _ptr(p.tile_expert), _ptr(p.tile_row0),
        _ptr(p.order), _ptr(p.weights), c_int(p.max_tiles), c_int(p.top), c_int(n), c_int(hidden), c_int(ff),
        c_int(0 if weight_on_input else 1), _stream()), "moe_down")
