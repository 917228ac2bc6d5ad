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


# --------------------------------------------------------------------------- attention
def paged_attention_generic(out, q, q_row_stride, k_pages, v_pages, block_tables, token_req, positions,
                            nq, nkv, head_dim, scale, window=0) -> None:
    """Causal attention of every token over its request's pages (generic float-math kernel).

    ``q`` is any tensor whose row t holds the q heads at [t * q_row_stride + h * D]."""
    _dev(out, q, k_pages, v_pages, block_tables, token_req, positions)
    n = out.shape[0]
    _need(out.shape == (n, nq * head_dim) and out.dtype == q.dtype, "out must be [tokens, nq * D] of q's type")
    _need(q.numel() >= (n - 1) * q_row_stride + nq * head_dim if n else True, "q is too small for its stride")
    _need(nkv > 0 and nq % nkv == 0, "q heads must be a multiple of kv heads")
    _need(head_dim <= 512, "head size above 512 is not supported")
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
           c_int(nq), c_int(nkv), c_int(head_dim), c_float(scale), c_int(window or 0), _stream()),
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


def attn_prefill_mfma(out, q, q_row_stride, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work, n_work,
                      nq, nkv, head_dim, scale, window=0) -> None:
    """Causal attention of prompt portions.  ``work`` is int32 [n_work, 3]: (request index, first row
    of a group, first row of a second group of the same request or -1), see ``attn_prefill_geometry``;
    every row of every request must be in exactly one group.  Pairing a group that sees many keys with
    one that sees few gives all blocks the same amount of work."""
    page_size = _attn_common(out, q, q_row_stride, k_pages, v_pages, block_tables, cu_seqlens, context_lens, work,
                             nq, nkv, head_dim)
    _need(work.numel() >= 3 * n_work, "work list shorter than n_work")
    lib = _attention_library(head_dim)
    _check(
        lib.jv_attn_prefill(_ptr(out), _ptr(q), c_longlong(q_row_stride), _ptr(k_pages), _ptr(v_pages),
                            _ptr(block_tables), c_int(block_tables.shape[1]), _ptr(cu_seqlens), _ptr(context_lens),
                            _ptr(work), c_int(n_work), c_int(page_size), c_int(nq), c_int(nkv), c_float(scale),
                            c_int(window or 0), _stream()),
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
                     nq, nkv, head_dim, scale, window=0, num_splits=1, scratch=None) -> None:
    """Attention of single decoded tokens.  ``work`` is int32 [n_work]: indices of the requests
    (each with exactly one token in this step); None: the step holds decoded tokens only, request
    r = 0 .. n_work-1 has its token in row r (the kernel then has nothing to look up before its
    loads start).  With ``num_splits`` > 1 a request's keys are shared out to that many blocks and
    ``scratch`` (float32, ``attn_decode_scratch_floats`` entries) holds their partial results."""
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
                           _stream()),
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
