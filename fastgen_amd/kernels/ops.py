"""Python faces of the HIP kernels.

Every function checks on the host that the operands have the shapes, dtypes
and strides the kernel and its grid assume, then launches on the current
stream of the tensors' device.  Nothing here runs on the CPU: a tensor that
is not on a GPU is refused.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
import os
from typing import Dict, Optional, Tuple

import numpy as np

import torch

from . import _lib

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelArgumentError(ValueError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelArgumentError(f"dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelArgumentError(msg)


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        _need(t.is_cuda, "fastgen_amd kernels run on the GPU only; got a tensor on " + str(t.device))
        dev = dev or t.device
        _need(t.device == dev, "operands live on different devices")


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # the stream's handle without a Stream object


def _stream(t: torch.Tensor) -> ctypes.c_void_p:
    """The device's current stream (a few hundred launches a step ask for it)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def upload(values, dtype: torch.dtype, device: torch.device | str) -> torch.Tensor:
    """``values`` (a numpy array or nested lists) on the device, through pinned host memory and a
    copy that does not make the host wait for the work already queued on the stream: a step can be
    prepared while the step before it runs.  (The pinned block goes back to torch's host allocator,
    which hands it out again only after the copy has happened.)"""
    src = torch.from_numpy(values) if isinstance(values, np.ndarray) else torch.tensor(values, dtype=dtype)
    if src.dtype != dtype:
        src = src.to(dtype)
    staged = torch.empty(src.shape, dtype=dtype, pin_memory=True)
    staged.copy_(src)
    return staged.to(device, non_blocking=True)


def _check(status: int, what: str) -> None:
    if status == 1:
        raise KernelArgumentError(f"{what}: the kernel refuses these sizes or dtypes")
    if status != 0:
        raise RuntimeError(f"{what}: launch failed (status {status})")


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be contiguous int32")
    if n is not None:
        _need(t.numel() >= n, f"{name} holds {t.numel()} entries, {n} are needed")


# --------------------------------------------------------------------- rows
def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[tokens[t]] * scale as fp32 (``fastgen/forward.py:406-409``, which has no scale)."""
    _gpu(table, tokens, out)
    n = tokens.numel()
    _need(table.dim() == 2 and table.is_contiguous(), "table must be contiguous [vocab, dim]")
    _i32(tokens, "tokens")
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (n, table.shape[1]),
          "out must be contiguous float32 [n_tokens, dim]")
    st = _lib.load("rows").fg_embed(
        _ptr(table), _code(table), _ptr(tokens), _ptr(out), n, table.shape[1], table.shape[0],
        ctypes.c_float(scale), _stream(out))
    _check(st, "embed")
    return out


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h += delta`` (fp32 residual stream), ``out = rmsnorm(h) * weight``.

    ``delta`` is ``[T, dim]`` of ``out``'s dtype, or fp32 ``[S, T, dim]``: partial
    sums of a matrix product whose k range was cut, added in order.  With
    ``rows`` only those rows of ``h`` are normed, into consecutive rows of
    ``out``, and ``h`` is left unchanged.  Norm as in
    ``fastgen/kernels/rmsnorm.py:33-60``.
    """
    _gpu(h, delta, weight, out, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [T, dim]")
    T, dim = h.shape
    n_rows = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, "rows")
    _need(weight.shape == (dim,) and weight.is_contiguous(), "weight must be [dim]")
    _need(out.is_contiguous() and out.shape == (n_rows, dim), "out must be contiguous [rows, dim]")
    parts, n_parts, part_stride = None, 0, 0
    if delta is not None and delta.dim() == 3:
        _need(delta.dtype == torch.float32 and delta.shape[1:] == h.shape and delta.stride(2) == 1
              and delta.stride(1) == dim, "partial sums must be float32 [S, T, dim] with contiguous rows")
        parts, n_parts, part_stride, delta = delta, delta.shape[0], delta.stride(0), None
    elif delta is not None:
        _need(delta.shape == h.shape and delta.is_contiguous() and delta.dtype == out.dtype,
              "delta must be contiguous, shaped like h, of out's dtype")
    st = _lib.load("rows").fg_add_rmsnorm(
        _ptr(h), _ptr(delta), _ptr(parts), n_parts, ctypes.c_longlong(part_stride), _ptr(weight), _ptr(out),
        _ptr(rows), n_rows, dim, ctypes.c_float(eps), _code(out), _code(weight), _stream(out))
    _check(st, "add_rmsnorm")
    return out


def _delta_args(h: torch.Tensor, delta: Optional[torch.Tensor], what: str):
    """C arguments (delta, dtype code, parts, n_parts, part stride) for what is to be added to the fp32
    stream ``h``: nothing, rows ``[T, dim]``, or fp32 partial sums ``[S, T, dim]``."""
    if delta is None:
        return _ptr(None), F32, _ptr(None), 0, ctypes.c_longlong(0)
    if delta.dim() == 3:
        _need(delta.dtype == torch.float32 and delta.shape[1:] == h.shape and delta.stride(2) == 1
              and delta.stride(1) == h.shape[1], f"{what}: partial sums must be float32 [S, T, dim] with contiguous rows")
        return _ptr(None), F32, _ptr(delta), delta.shape[0], ctypes.c_longlong(delta.stride(0))
    _need(delta.shape == h.shape and delta.is_contiguous(), f"{what}: delta must be contiguous and shaped like h")
    return _ptr(delta), _code(delta), _ptr(None), 0, ctypes.c_longlong(0)


def stream_add(h: torch.Tensor, delta: Optional[torch.Tensor], again: Optional[torch.Tensor],
               row: Optional[torch.Tensor]) -> torch.Tensor:
    """``h = ((h + delta) + again) + row`` in place on the fp32 stream ``h [T, dim]``, in that order:
    ``delta`` as :func:`add_rmsnorm` takes it, ``again`` fp32 ``[T, dim]``, ``row`` fp32 ``[dim]`` for
    every token.  Each may be None."""
    _gpu(h, delta, again, row)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [T, dim]")
    T, dim = h.shape
    if again is not None:
        _need(again.dtype == torch.float32 and again.shape == h.shape and again.is_contiguous(),
              "again must be contiguous float32, shaped like h")
    if row is not None:
        _need(row.dtype == torch.float32 and row.shape == (dim,) and row.is_contiguous(), "row must be float32 [dim]")
    st = _lib.load("rows").fg_stream_add(_ptr(h), *_delta_args(h, delta, "stream_add"), _ptr(again), _ptr(row), T, dim,
                                         _stream(h))
    _check(st, "stream_add")
    return h


def add_rows(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``a + b`` of two ``[T, dim]`` tensors of one dtype as fp32 ``[1, T, dim]``: two sublayers' outputs
    as the one sum that a norm adds to the stream."""
    _gpu(a, b)
    _need(a.dim() == 2 and a.shape == b.shape and a.dtype == b.dtype and a.is_contiguous() and b.is_contiguous(),
          "a and b must be contiguous [T, dim] of one dtype")
    out = torch.empty((1, *a.shape), dtype=torch.float32, device=a.device)
    st = _lib.load("rows").fg_add_rows(_ptr(a), _ptr(b), _ptr(out), ctypes.c_longlong(a.numel()), _code(a), _stream(a))
    _check(st, "add_rows")
    return out


def gate_mul(x: torch.Tensor, gate: torch.Tensor, sigmoid: bool = True) -> torch.Tensor:
    """``x *= sigmoid(gate)`` in place (``x *= gate`` with ``sigmoid=False``); ``x`` and ``gate`` are
    ``[T, width]`` with unit column stride and row strides of their own."""
    _gpu(x, gate)
    _need(x.dim() == 2 and gate.dim() == 2 and x.shape[0] == gate.shape[0] and gate.shape[1] >= x.shape[1]
          and x.dtype == gate.dtype and x.stride(1) == 1 and gate.stride(1) == 1,
          "x [T, width] and gate [T, >= width] must share a dtype and have unit column stride")
    st = _lib.load("rows").fg_gate_mul(_ptr(x), x.stride(0), _ptr(gate), gate.stride(0), x.shape[0], x.shape[1],
                                       int(sigmoid), _code(x), _stream(x))
    _check(st, "gate_mul")
    return x


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm over the last dimension of a contiguous tensor."""
    _gpu(x, weight, out)
    _need(x.is_contiguous(), "x must be contiguous")
    dim = x.shape[-1]
    out = torch.empty_like(x) if out is None else out
    _need(out.shape == x.shape and out.dtype == x.dtype and out.is_contiguous(), "out must match x")
    _need(weight.shape == (dim,) and weight.is_contiguous(), "weight must be [dim]")
    st = _lib.load("rows").fg_rmsnorm(
        _ptr(x), _ptr(weight), _ptr(out), x.numel() // dim, dim, ctypes.c_float(eps), _code(x),
        _code(weight), _stream(out))
    _check(st, "rmsnorm")
    return out


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of a gate and an up matrix ``[hidden, dim]`` as one matrix
    ``[2*hidden, dim]`` in groups of 8: rows ``16k..16k+7`` are gate rows
    ``8k..8k+7``, rows ``16k+8..16k+15`` the up rows of the same channels.  One
    16-row tile of a product with it holds both halves of 8 channels, so
    ``silu(gate) * up`` can be applied where the tile is stored."""
    hidden, dim = gate.shape
    _need(up.shape == gate.shape and hidden % 8 == 0,
          f"gate and up must have the same shape and a row count that is a multiple of 8 (got {hidden})")
    return torch.stack([gate.reshape(hidden // 8, 8, dim), up.reshape(hidden // 8, 8, dim)], dim=1).reshape(
        2 * hidden, dim)


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` of ``[T, 2*hidden]`` whose columns are interleaved as
    :func:`interleave_gate_up` orders the matrix rows; fp32 inside."""
    _gpu(gate_up, out)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 16 == 0,
          "gate_up must be contiguous [T, 2*hidden] with hidden a multiple of 8")
    T, hidden = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, hidden), dtype=gate_up.dtype, device=gate_up.device) if out is None else out
    _need(out.shape == (T, hidden) and out.dtype == gate_up.dtype and out.is_contiguous(), "out must be [T, hidden]")
    st = _lib.load("rows").fg_silu_mul(_ptr(gate_up), _ptr(out), T, hidden, _code(out), _stream(out))
    _check(st, "silu_mul")
    return out


def gelu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``gelu_tanh(gate) * up`` of ``[T, 2*hidden]`` laid out as :func:`silu_mul` takes it;
    ``gelu_tanh(g) = 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))``, fp32 inside."""
    _gpu(gate_up, out)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 16 == 0,
          "gate_up must be contiguous [T, 2*hidden] with hidden a multiple of 8")
    T, hidden = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, hidden), dtype=gate_up.dtype, device=gate_up.device) if out is None else out
    _need(out.shape == (T, hidden) and out.dtype == gate_up.dtype and out.is_contiguous(), "out must be [T, hidden]")
    st = _lib.load("rows").fg_gelu_mul(_ptr(gate_up), _ptr(out), T, hidden, _code(out), _stream(out))
    _check(st, "gelu_mul")
    return out


@dataclass
class PostNormed:
    """A sublayer's output that is RMS-normed (``weight``, ``eps``) before it is added to the residual
    stream: ``rows`` is ``[T, dim]`` of the activation dtype or fp32 ``[S, T, dim]`` partial sums.  A norm
    on the stream takes it where it takes rows to be added (:func:`post_add_rmsnorm`)."""

    rows: torch.Tensor
    weight: torch.Tensor
    eps: float
    bias: Optional[torch.Tensor] = None  # fp32 [dim]: added to the rows before their norm (a projection's bias)


def post_add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], post_weight: Optional[torch.Tensor],
                     post_eps: float, weight: Optional[torch.Tensor], eps: float, out: Optional[torch.Tensor],
                     rows: Optional[torch.Tensor] = None, delta_bias: Optional[torch.Tensor] = None
                     ) -> Optional[torch.Tensor]:
    """``h += rmsnorm(delta + delta_bias) * post_weight`` on the fp32 stream ``h [T, dim]`` and, with ``weight``,
    ``out = rmsnorm(h) * weight``: the norm behind a sublayer, the addition and the norm before the next
    one in one pass, all in fp32.  ``delta`` as :func:`add_rmsnorm` takes it; None: nothing is added.  With
    ``out`` but without ``weight`` the stream's rows themselves are stored, rounded to ``out``'s dtype (what a
    sublayer reads that takes the stream un-normed).  With ``rows`` only those rows are computed, into
    consecutive rows of ``out``, and ``h`` is left as it was."""
    _gpu(h, delta, post_weight, weight, out, rows, delta_bias)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [T, dim]")
    T, dim = h.shape
    n_rows = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, "rows")
    _need(delta is None or post_weight is not None, "rows that are added are normed: post_weight is missing")
    _need(delta is not None or out is not None, "nothing to add and nothing to store")
    if post_weight is not None:
        _need(post_weight.shape == (dim,) and post_weight.is_contiguous(), "post_weight must be [dim]")
    if weight is not None:
        _need(weight.shape == (dim,) and weight.is_contiguous()
              and (post_weight is None or weight.dtype == post_weight.dtype), "weight must be [dim], of post_weight's dtype")
    if out is not None:
        _need(out.is_contiguous() and out.shape == (n_rows, dim), "out must be contiguous [rows, dim]")
    else:
        _need(weight is None and rows is None, "a norm or a gathered call needs out")
    _f32_vec(delta_bias, dim, "delta_bias")
    act = out.dtype if out is not None else (delta.dtype if delta.dim() == 2 else torch.float32)
    d_ptr, d_code, parts, n_parts, part_stride = _delta_args(h, delta, "post_add_rmsnorm")
    if delta is not None and delta.dim() == 2:
        _need(delta.dtype == act, "delta must have out's dtype")
    w_any = post_weight if post_weight is not None else weight
    st = _lib.load("rows").fg_post_add_rmsnorm(
        _ptr(h), d_ptr, parts, n_parts, part_stride, _ptr(post_weight), ctypes.c_float(post_eps), _ptr(weight),
        _ptr(out), _ptr(rows), n_rows, dim, ctypes.c_float(eps), _DTYPE_CODE[act],
        _code(w_any) if w_any is not None else F32, _ptr(delta_bias), _stream(h))
    _check(st, "post_add_rmsnorm")
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x = cap * tanh(x / cap)`` in place on contiguous fp32."""
    _gpu(x)
    _need(x.dtype == torch.float32 and x.is_contiguous() and cap > 0, "x must be contiguous float32, cap positive")
    st = _lib.load("rows").fg_softcap(_ptr(x), ctypes.c_longlong(x.numel()), ctypes.c_float(cap), _stream(x))
    _check(st, "softcap")
    return x


# ------------------------------------------------------------ rope + kv write
def scale_logits(x: torch.Tensor, factor: float) -> torch.Tensor:
    """``x *= factor`` in place on contiguous fp32."""
    _gpu(x)
    _need(x.dtype == torch.float32 and x.is_contiguous(), "x must be contiguous float32")
    _check(_lib.load("rows").fg_scale(_ptr(x), ctypes.c_longlong(x.numel()), ctypes.c_float(factor), _stream(x)), "scale_logits")
    return x


def rope_table(positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """``[T, n_freqs, 2]`` fp32: cos and sin of ``float(pos) * freqs[i]``, for all
    layers of a step that rotate with the same frequencies."""
    _gpu(positions, freqs)
    _i32(positions, "positions")
    _need(freqs.dtype == torch.float32 and freqs.is_contiguous(), "freqs must be contiguous float32")
    T, n = positions.numel(), freqs.numel()
    table = torch.empty((T, n, 2), dtype=torch.float32, device=positions.device)
    st = _lib.load("rope_kv").fg_rope_table(_ptr(positions), _ptr(freqs), _ptr(table), T, n, _stream(table))
    _check(st, "rope_table")
    return table


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, freqs: Optional[torch.Tensor],
                  slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
                  rotary_dim: int, write_kv: bool = True, table: Optional[torch.Tensor] = None,
                  v_col: Optional[int] = None) -> None:
    """Rotate q and k of ``qkv [T, (H+2KV)*hd]`` in place and store k, v at
    ``slots`` of the paged cache (K pages ``[n_pages, KV, P, hd]``, V pages
    ``[n_pages, KV, hd, P]``).  ``kernels/rope.py:56-89``, ``forward.py:449-460``.
    ``v_col``: the column at which a row's values begin (default: behind the keys);
    ``n_heads * head_dim`` makes a token's value its key before the rotation.
    """
    _gpu(qkv, positions, freqs, slots, k_pages, v_pages)
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "qkv must be [T, width] with unit column stride")
    T = qkv.shape[0]
    v_col = (n_heads + n_kv) * head_dim if v_col is None else int(v_col)
    width = max((n_heads + n_kv) * head_dim, v_col + n_kv * head_dim) if write_kv else n_heads * head_dim
    _need(qkv.shape[1] >= width, f"qkv rows hold {qkv.shape[1]} elements, {width} are needed")
    _need(v_col >= n_heads * head_dim and v_col % 8 == 0, "the values begin behind the queries, at a multiple of 8")
    _i32(positions, "positions", T)
    _need(head_dim % 2 == 0 and 0 <= rotary_dim <= head_dim and rotary_dim % 2 == 0,
          "head_dim and rotary_dim must be even and rotary_dim <= head_dim")
    if rotary_dim and table is None:
        _need(freqs is not None and freqs.dtype == torch.float32 and freqs.is_contiguous()
              and freqs.numel() >= rotary_dim // 2, "freqs must be float32 [rotary_dim/2]")
    if rotary_dim and table is not None:
        _need(table.dtype == torch.float32 and table.is_contiguous() and table.shape == (T, rotary_dim // 2, 2),
              "table must be float32 [T, rotary_dim/2, 2]")
    page_size = 1
    if write_kv:
        _need(slots is not None and k_pages is not None and v_pages is not None, "cache operands missing")
        _i32(slots, "slots", T)
        _need(k_pages.dim() == 4 and k_pages.is_contiguous() and k_pages.dtype == qkv.dtype
              and k_pages.shape[1] == n_kv and k_pages.shape[3] == head_dim,
              "k_pages must be contiguous [n_pages, KV, P, hd] of qkv's dtype")
        page_size = k_pages.shape[2]
        _need(v_pages.is_contiguous() and v_pages.dtype == qkv.dtype
              and v_pages.shape == (k_pages.shape[0], n_kv, head_dim, page_size),
              "v_pages must be contiguous [n_pages, KV, hd, P] of qkv's dtype")
    st = _lib.load("rope_kv").fg_rope_kv_write(
        _ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(freqs), _ptr(table if rotary_dim else None), _ptr(slots),
        _ptr(k_pages), _ptr(v_pages),
        T, n_heads, n_kv, head_dim, rotary_dim, page_size, int(write_kv), v_col, _code(qkv), _stream(qkv))
    _check(st, "rope_kv_write")


# ------------------------------------------------------------------ attention
def _sinks_ok(sinks: Optional[torch.Tensor], n_heads: int) -> None:
    if sinks is not None:
        _need(sinks.dtype == torch.float32 and sinks.is_contiguous() and sinks.shape == (n_heads,),
              "sinks must be contiguous float32 [n_heads]")


def paged_attention_general(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                            block_table: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                            n_heads: int, scale: float, window: int = 0,
                            sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of every token over its sequence's cached keys.

    ``q`` is ``[T, >= H*hd]`` (the first ``H*hd`` columns are the query heads;
    it may be a qkv buffer), ``out`` is ``[T, H*hd]``.  ``forward.py:176-258``.
    ``sinks``: fp32 ``[H]``; head ``h``'s softmax has one more term ``exp(sinks[h])`` in its
    denominator, which brings no value.  ``window`` > 0: a token at position ``p`` sees the keys
    ``p - window + 1 .. p``; ``window`` < 0: the keys up to ``p`` of its own block of ``-window`` positions,
    blocks counted from position 0 of the sequence (:func:`block_mask`); 0: every key up to ``p``.
    """
    _gpu(q, out, k_pages, v_pages, block_table, seq_of_token, positions, sinks)
    _sinks_ok(sinks, n_heads)
    T = q.shape[0]
    _need(k_pages.dim() == 4 and k_pages.is_contiguous(), "k_pages must be contiguous [n_pages, KV, P, hd]")
    n_pages, n_kv, page_size, hd = k_pages.shape
    _need(v_pages.shape == (n_pages, n_kv, hd, page_size) and v_pages.is_contiguous(),
          "v_pages must be contiguous [n_pages, KV, hd, P]")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * hd, "q must be [T, >= H*hd]")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape == (T, n_heads * hd), "out must be [T, H*hd]")
    _need(q.dtype == out.dtype == k_pages.dtype == v_pages.dtype, "q, out and the cache must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1,
          "block_table must be int32 [B, max_pages]")
    _i32(seq_of_token, "seq_of_token", T)
    _i32(positions, "positions", T)
    _need(n_heads % n_kv == 0, "the number of heads must be a multiple of the number of kv heads")
    _need(hd % 8 == 0 and hd <= 512, f"head size {hd} is not supported (multiple of 8, at most 512)")
    _need(page_size % 8 == 0, f"page size {page_size} is not supported (multiple of 8)")
    st = _lib.load("attention").fg_paged_attention_general_sink(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        block_table.stride(0), _ptr(seq_of_token), _ptr(positions), T, n_heads, n_kv, hd, page_size,
        ctypes.c_float(scale), int(window or 0), _ptr(sinks), _code(q), _stream(q))
    _check(st, "paged_attention_general")
    return out


def block_mask(size: Optional[int]) -> int:
    """The ``window`` argument of the attention functions for a mask of blocks of ``size`` positions: a token
    sees the keys before it (and itself) inside its own block, blocks counted from position 0."""
    return -int(size) if size else 0


MFMA_MAX_HEAD_DIM = 256

_n_cus: Optional[int] = None


def compute_units() -> int:
    """Compute units of the current device (asked once)."""
    global _n_cus
    if _n_cus is None:
        _n_cus = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
    return _n_cus


def _split_target_blocks() -> int:
    """Workgroups wanted for the decode attention kernel: one per compute unit measured best (half as many
    to eight times as many tried at batch 1, 8 and 64).  The splits' partial results are merged by a second
    kernel: merging them in the split that finishes last needs device-scope fences, which on a GPU of
    several dies cost more than the launch they save (measured)."""
    env = os.environ.get("FG_SPLIT_TARGET")
    return int(env) if env else compute_units()


# a chunk of the decode attention's key ranges is a multiple of this many 64-key tiles (one a wave)
_SPLIT_MIN_TILES = int(os.environ.get("FG_SPLIT_MIN_TILES", 4))


def _mfma_attention(head_dim: int, exact: bool = False):
    """The matrix-core attention library for this head size: the plain build, or the one whose softmax
    weights keep 16 significant bits (a model that asks for it loads only that one)."""
    return _lib.load(f"attention_mfma_exact@{head_dim}" if exact else f"attention_mfma@{head_dim}")


def attention_tile_rows(head_dim: int, small: bool = False, exact: bool = False) -> int:
    """Query rows of one item of the tile kernel for this head size: of its larger form (128 rows up to
    head size 128), or of the form with ``small`` items (64 rows, more and lighter workgroups)."""
    return int(_mfma_attention(head_dim, exact).fg_attn_tile_rows(int(small)))


def attention_items(q_lens, q_start, n_cached, group_size: int, tile_rows: int = 64):
    """Cut the step's sequences into items for the MFMA kernels.

    Returns two int32 arrays ``[n, 4]`` of (sequence, first flat token, tokens,
    position of the first token): items of at most 16 rows for the split
    kernel (decoded tokens and very short portions) and items of at most
    ``tile_rows`` rows for the tile kernel, those with the most keys first (the
    kernel's workgroups start in that order, so short items fill in behind long
    ones).
    """
    small, big = [], []
    per_tile = max(1, tile_rows // group_size)
    for b, n in enumerate(q_lens):
        n, s, c = int(n), int(q_start[b]), int(n_cached[b])
        if n * group_size <= 16:
            small.append((b, s, n, c))
        else:
            big.extend((b, s + i, min(per_tile, n - i), c + i) for i in range(0, n, per_tile))
    big.sort(key=lambda it: -(it[3] + it[2]))  # the longest key ranges start first
    as_arr = lambda x: np.asarray(x, dtype=np.int32).reshape(-1, 4)
    return as_arr(small), as_arr(big)


def attention_chunks_for(n_items: int, n_kv: int) -> int:
    """Length of the split kernel's chunk list for ``n_items`` items: enough chunks for a few
    workgroups per compute unit, and at least two an item so that a long sequence among short
    ones can be cut."""
    return max(-(-_split_target_blocks() // n_kv) + n_items, 2 * n_items)


def _plan_ints(lib, max_chunks: int) -> int:
    lib.fg_attn_plan_ints.restype = ctypes.c_longlong
    return int(lib.fg_attn_plan_ints(max_chunks))


def attention_plan(items: torch.Tensor, n_items: int, max_chunks: int, head_dim: int, window: int = 0,
                   min_tiles: int = 4, exact: bool = False) -> torch.Tensor:
    """Cuts the key ranges of ``items`` (device int32 ``[n_items, 4]``, 16-byte aligned) into chunks of
    the same number of 64-key tiles, a multiple of ``min_tiles``, on the device: a captured step cuts
    anew for the lengths of every replay.  The int32 plan that :func:`paged_attention_mfma` takes."""
    _gpu(items)
    _i32(items, "items")
    _need(items.data_ptr() % 16 == 0 and items.numel() >= 4 * n_items > 0, "items must be [n, 4], 16-byte aligned")
    _need(max_chunks >= 2 * n_items and min_tiles >= 1, "max_chunks must be at least twice the number of items")
    lib = _mfma_attention(head_dim, exact)  # the plan is the same for every head size and build
    plan = torch.empty(_plan_ints(lib, max_chunks), dtype=torch.int32, device=items.device)
    _check(lib.fg_attn_plan(_ptr(items), n_items, int(window or 0), max_chunks, min_tiles, _ptr(plan),
                            _stream(items)), "attn_plan")
    return plan


_ONE_STREAM = bool(os.environ.get("FG_ONE_STREAM"))  # no kernel runs beside another
_second: Dict[int, "torch.cuda.Stream"] = {}


def _second_stream(device) -> "torch.cuda.Stream":
    """A stream of the default priority beside the current one, one a device, made at first use."""
    index = torch.device(device).index
    index = torch.cuda.current_device() if index is None else index
    if index not in _second:
        _second[index] = torch.cuda.Stream(device)
    return _second[index]


def paged_attention_mfma(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                         block_table: torch.Tensor, small_items: Optional[torch.Tensor],
                         big_items: Optional[torch.Tensor], n_heads: int, scale: float, window: int = 0,
                         plan: Optional[torch.Tensor] = None, max_chunks: Optional[int] = None,
                         min_tiles: int = 4, max_rows: int = 16, tile_rows: Optional[int] = None,
                         exact_weights: bool = False, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 attention on the matrix cores.  ``small_items`` / ``big_items`` are
    device int32 ``[n, 4]`` lists from :func:`attention_items` (16-byte aligned);
    every query token of the step must be covered by exactly one item.
    ``plan``: :func:`attention_plan` of the small items with this ``max_chunks``
    and ``window`` (made here if not given).  ``max_rows``: no small item has
    more rows (tokens times query heads per kv head) than this.  ``tile_rows``: the
    rows the big items were cut for (:func:`attention_tile_rows`; default: the larger form's).
    With items of both kinds the tile kernel runs on a second stream beside the split kernel and
    the current stream waits for it before this returns (not while a graph is captured, not with
    ``FG_ONE_STREAM=1``).  ``exact_weights``: the build of the kernels in which the softmax weights enter
    the product with the values as two bfloat16 terms (16 significant bits).  ``sinks``: as
    :func:`paged_attention_general`."""
    _gpu(q, out, k_pages, v_pages, block_table, small_items, big_items, plan, sinks)
    _sinks_ok(sinks, n_heads)
    n_pages, n_kv, page_size, hd = k_pages.shape
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16
          and v_pages.dtype == torch.bfloat16, "the MFMA attention kernels take bfloat16")
    _need(hd % 16 == 0 and hd <= MFMA_MAX_HEAD_DIM, f"head size {hd}: multiples of 16 up to {MFMA_MAX_HEAD_DIM}")
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and v_pages.shape == (n_pages, n_kv, hd, page_size),
          "k_pages [n_pages, KV, P, hd] and v_pages [n_pages, KV, hd, P] must be contiguous")
    _need(n_heads % n_kv == 0 and page_size % 8 == 0, "heads must be a multiple of kv heads, pages of 8 tokens")
    _need(scale > 0, "the score scale must be positive")
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * hd and q.stride(0) % 8 == 0
          and q.data_ptr() % 16 == 0, "q must be [T, >= H*hd], rows 16-byte aligned")
    _need(out.shape == (T, n_heads * hd) and out.stride(1) == 1 and out.stride(0) % 4 == 0, "out must be [T, H*hd]")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1,
          "block_table must be int32 [B, max_pages]")
    lib = _mfma_attention(hd, exact_weights)
    G = n_heads // n_kv
    beside = None
    if (small_items is not None and small_items.numel() and big_items is not None and big_items.numel()
            and not _ONE_STREAM and not torch.cuda.is_current_stream_capturing()):
        # a step with both kinds of items (prompt portions beside decoded tokens): the two kernels write
        # different rows of `out`, one is bound by the matrix cores and one by memory, so the tile kernel
        # runs on a second stream beside the split kernel (3 % of a continuous-batching run)
        beside = _second_stream(q.device)
        beside.wait_event(torch.cuda.current_stream(q.device).record_event())
    if small_items is not None and small_items.numel():
        _need(G <= 16 and 1 <= max_rows <= 16, "the split kernel takes at most 16 rows an item")
        _i32(small_items, "small_items")
        _need(small_items.data_ptr() % 16 == 0, "items must be 16-byte aligned")
        n = small_items.numel() // 4
        if max_chunks is None:
            max_chunks = attention_chunks_for(n, n_kv)
        _need(2 * n <= max_chunks <= 65535, "the chunk list holds at least two chunks an item and at most 65535")
        if plan is None:
            plan = attention_plan(small_items, n, max_chunks, hd, window, min_tiles, exact_weights)
        _need(plan.dtype == torch.int32 and plan.numel() == _plan_ints(lib, max_chunks),
              "the plan does not fit the items and max_chunks")
        part_o = torch.empty((max_chunks * n_kv * 16, hd), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((max_chunks * n_kv * 16, 2), dtype=torch.float32, device=q.device)
        st = lib.fg_attn_split_sink(
            _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            block_table.stride(0), _ptr(plan), n, max_chunks, max_rows, _ptr(part_o), _ptr(part_ml), n_heads, n_kv, hd,
            page_size, ctypes.c_float(scale), int(window or 0), _ptr(sinks), _stream(q))
        _check(st, "attn_split")
    if big_items is not None and big_items.numel():
        tile_rows = attention_tile_rows(hd, False, exact_weights) if tile_rows is None else int(tile_rows)
        _need(tile_rows in (attention_tile_rows(hd, False, exact_weights), attention_tile_rows(hd, True, exact_weights)),
              "tile_rows is no form of the tile kernel")
        _need(G <= tile_rows, "too many query heads per kv head for the tile kernel")
        _i32(big_items, "big_items")
        _need(big_items.data_ptr() % 16 == 0, "items must be 16-byte aligned")
        st = lib.fg_attn_tile_sink(
            _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            block_table.stride(0), _ptr(big_items), big_items.numel() // 4, tile_rows, n_heads, n_kv, hd, page_size,
            ctypes.c_float(scale), int(window or 0), _ptr(sinks),
            ctypes.c_void_p(beside.cuda_stream) if beside else _stream(q))
        _check(st, "attn_tile")
        if beside is not None:
            torch.cuda.current_stream(q.device).wait_event(beside.record_event())
    return out


def paged_attention(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                    group, ctx, n_heads: int, scale: float, window: int = 0,
                    exact_weights: bool = False, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention for one step: picks the kernel for the step's dtype and shape.
    ``exact_weights``: see :func:`paged_attention_mfma` (the general kernel's weights are fp32 anyway).

    ``group`` carries the block table of the layer's cache group, ``ctx`` the
    step's per-token vectors (``fastgen_amd.engine.context``).  bfloat16 with a
    head size in steps of 16 up to 256 and at most 16 query heads per kv head
    runs on the matrix cores; everything else (float32 always) runs the general
    kernel.
    """
    n_kv, hd = k_pages.shape[1], k_pages.shape[3]
    G = n_heads // n_kv
    if q.dtype != torch.bfloat16 or hd % 16 or hd > MFMA_MAX_HEAD_DIM or G > 16:
        return paged_attention_general(q, out, k_pages, v_pages, group.block_table, ctx.seq_of_token,
                                       ctx.positions, n_heads, scale, window, sinks)
    items_key = ("attention_items", G, hd, n_kv)  # (how a step is cut into items depends on all three)
    plan = ctx.scratch.get(items_key)
    if plan is None:
        if ctx.seq_records is not None and int(ctx.q_lens.max()) * G <= 16:
            # every sequence is one item of the split kernel: its records are in the step's buffer
            # already (and are refreshed with it when the step is a replayed graph)
            plan = (ctx.seq_records, None, ctx.n_seqs, None)
        else:
            tile_rows = attention_tile_rows(hd, False, exact_weights)
            small, big = attention_items(ctx.q_lens, ctx.q_start_host, ctx.n_cached, G, tile_rows)
            if 0 < len(big) * n_kv <= compute_units() // 2 and attention_tile_rows(hd, True, exact_weights) < tile_rows:
                # so few items that half the compute units would stand idle: items of half the rows, whose
                # lighter workgroups share a unit (prompt portions of up to 512 tokens: 11.6 / 17.6 us
                # against 14.1 / 19.5 at 256 / 512 tokens; equal at 1,024, slower beyond)
                tile_rows = attention_tile_rows(hd, True, exact_weights)
                small, big = attention_items(ctx.q_lens, ctx.q_start_host, ctx.n_cached, G, tile_rows)
            both = upload(np.concatenate([small, big]).reshape(-1), torch.int32, q.device)
            plan = (both[: small.size] if small.size else None, both[small.size:] if big.size else None, len(small),
                    tile_rows)
        ctx.scratch[items_key] = plan
    small_d, big_d, n_small, tile_rows = plan
    chunks = split_plan = None
    if n_small:
        # how the items' key ranges are cut depends on the window: layers with the same one share the cut
        chunks = attention_chunks_for(n_small, n_kv)
        key = ("attention_plan", G, int(window or 0), chunks)
        split_plan = ctx.scratch.get(key)
        if split_plan is None:
            split_plan = ctx.scratch[key] = attention_plan(small_d, n_small, chunks, hd, window, _SPLIT_MIN_TILES,
                                                           exact_weights)
    # rows of the largest small item: one token a sequence in a decode step (also a captured one)
    rows = G * int(ctx.q_lens.max()) if big_d is None else 16
    return paged_attention_mfma(q, out, k_pages, v_pages, group.block_table, small_d, big_d, n_heads, scale,
                                window, split_plan, chunks, max_rows=min(16, rows), tile_rows=tile_rows,
                                exact_weights=exact_weights, sinks=sinks)


# ----------------------------------------------------------------------- gemm
def gemm_nt(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
            out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x @ w.T`` with ``w [N, K]``, by the engine's own fp32-FMA kernel (sum
    over k in ascending order; a row's result does not depend on the others)."""
    _gpu(x, w, out)
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], "x [M,K] and w [N,K] must share K")
    _need(x.stride(1) == 1 and w.stride(1) == 1, "x and w need unit column stride")
    _need(x.dtype == w.dtype, "x and w must share a dtype")
    M, K = x.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "out must be [M, N]")
    for m0 in range(0, M, 65535 * 64):  # grid.y limit
        m1 = min(M, m0 + 65535 * 64)
        st = _lib.load("gemm").fg_gemm_nt(
            _ptr(x[m0:m1]), _ptr(w), _ptr(out[m0:m1]), m1 - m0, N, K, x.stride(0), w.stride(0), out.stride(0),
            _code(x), _code(out), _stream(out))
        _check(st, "gemm_nt")
    return out


SKINNY_MAX_ROWS = 128

# epilogue codes of the streaming and tiled products: store; silu(gate) * up; gelu_tanh(gate) * up
_GATED_CODE = {False: 0, None: 0, True: 1, "silu": 1, "gelu_tanh": 4}


def _gated_code(epilogue) -> int:
    """The kernels' code for a ``silu_mul_epilogue`` argument: False, True (SiLU), or the activation's name."""
    try:
        return _GATED_CODE[epilogue]
    except (KeyError, TypeError):
        raise KernelArgumentError(f"unknown gated epilogue {epilogue!r} (True, 'silu' or 'gelu_tanh')") from None


@dataclass
class PackedWeight:
    """A bfloat16 weight matrix ``[n, k]`` in the order in which the streaming products read it
    (:func:`pack_weight`): ``data [ceil(n / 16), ceil(k / 32), 64, 8]``, a block of 16 rows x 32 k as
    the 1 KB that a wave holds as one MFMA operand (lane ``16 g + r``: row ``r``, k ``8 g .. 8 g + 7``),
    rows and k padded with zeros.  A wave's load is then whole cache lines in a row; from a matrix
    stored row by row it is 16 pieces of half a line."""

    data: torch.Tensor
    n: int
    k: int

    @property
    def shape(self) -> Tuple[int, int]:
        return (self.n, self.k)

    @property
    def dtype(self) -> torch.dtype:
        return self.data.dtype

    def first_rows(self, n: int) -> "PackedWeight":
        """The matrix of the first ``n`` rows (a multiple of 16, or all): a view."""
        _need(0 < n <= self.n and (n % 16 == 0 or n == self.n), "a packed matrix is cut at multiples of 16 rows")
        return PackedWeight(self.data[: -(-n // 16)], n, self.k)


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """``w [n, k]`` (bfloat16) as :class:`PackedWeight`: a copy, on the device of ``w``."""
    _need(w.dim() == 2 and w.dtype == torch.bfloat16, "pack_weight takes a bfloat16 matrix")
    n, k = w.shape
    nb, ks = -(-n // 16), -(-k // 32)
    if (nb * 16, ks * 32) != (n, k):
        padded = w.new_zeros((nb * 16, ks * 32))
        padded[:n, :k] = w
        w = padded
    # [nb, r, ks, g, 8] -> [nb, ks, g, r, 8]
    data = w.view(nb, 16, ks, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(nb, ks, 64, 8)
    return PackedWeight(data, n, k)


def unpack_weight(p: PackedWeight) -> torch.Tensor:
    """The matrix ``[n, k]`` that :func:`pack_weight` was given."""
    nb, ks = p.data.shape[:2]
    w = p.data.view(nb, ks, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nb * 16, ks * 32)
    return w[: p.n, : p.k].contiguous()


def _weight_args(w, K: int, what: str):
    """C arguments (pointer, ldw) for the weight of a streaming product, a matrix or :class:`PackedWeight`
    (ldw = 0), checked against the k of x."""
    if isinstance(w, PackedWeight):
        _gpu(w.data)
        _need(w.data.dtype == torch.bfloat16 and w.data.is_contiguous() and w.k == K
              and w.data.shape == (-(-w.n // 16), -(-w.k // 32), 64, 8) and w.data.data_ptr() % 16 == 0,
              f"{what}: the packed weight does not fit x [M, {K}]")
        return _ptr(w.data), 0
    _gpu(w)
    _need(w.dim() == 2 and w.dtype == torch.bfloat16 and w.shape[1] == K, f"{what}: w must be bfloat16 [N, {K}]")
    _need(w.stride(1) == 1 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0, f"{what}: w needs 16-byte aligned rows")
    return _ptr(w), w.stride(0)


@dataclass
class ScaledRows:
    """Rows that are not yet divided by their root mean square: the true row ``t`` is
    ``rows[t] * rsqrt(sum(ssq[t]) / dim + eps)``.  For few rows the norm before a matrix product
    is folded into the products around it: the one before stores ``rows`` and the sums of squares
    of its workgroups' columns (:func:`gemm_skinny_residual`), the one after scales its result
    rows (``x @ w.T`` is linear in a row's scale)."""

    rows: torch.Tensor  # [T, dim] bfloat16
    ssq: torch.Tensor  # [T, n_parts] float32
    dim: int
    eps: float

    @property
    def shape(self):
        return self.rows.shape

    def materialize(self) -> torch.Tensor:
        """The rows themselves (a kernel of its own: for a consumer that does not take the pair)."""
        return scale_rows(self.rows, self.ssq, self.dim, self.eps)


def _row_scale_args(x, M: int):
    """C arguments (ssq, n_parts, dim, eps) for ``x`` a tensor or :class:`ScaledRows`."""
    if not isinstance(x, ScaledRows):
        return ctypes.c_void_p(0), 0, 0, ctypes.c_float(0.0)
    ssq = x.ssq
    _need(ssq.dtype == torch.float32 and ssq.is_contiguous() and ssq.dim() == 2 and ssq.shape[0] == M
          and ssq.is_cuda, "ssq must be contiguous float32 [M, n_parts] on the GPU")
    _need(x.dim > 0 and x.eps >= 0, "ScaledRows needs dim > 0 and eps >= 0")
    return _ptr(ssq), ssq.shape[1], int(x.dim), ctypes.c_float(x.eps)


def scale_rows(rows: torch.Tensor, ssq: torch.Tensor, dim: int, eps: float) -> torch.Tensor:
    """``rows[t] * rsqrt(sum(ssq[t]) / dim + eps)`` in the dtype of ``rows``."""
    _gpu(rows, ssq)
    _need(rows.dim() == 2 and rows.is_contiguous() and ssq.dim() == 2 and ssq.is_contiguous()
          and ssq.dtype == torch.float32 and ssq.shape[0] == rows.shape[0], "rows [T, D], ssq float32 [T, n_parts]")
    out = torch.empty_like(rows)
    st = _lib.load("rows").fg_scale_rows(_ptr(rows), _ptr(ssq), _ptr(out), rows.shape[0], rows.shape[1],
                                         ssq.shape[1], int(dim), ctypes.c_float(eps), _code(rows), _stream(rows))
    _check(st, "scale_rows")
    return out


def gemm_skinny_residual(x: torch.Tensor, w, h: torch.Tensor, norm_weight: torch.Tensor,
                         eps: float) -> ScaledRows:
    """For at most 16 rows: ``h += x @ w.T`` on the fp32 residual stream ``h [M, N]`` and, in the same
    kernel, what the RMSNorm that follows needs: ``h * norm_weight`` in bfloat16 and a sum of squares
    of ``h`` per row and workgroup (16 columns).  ``x`` may itself be :class:`ScaledRows`, ``w`` a
    matrix or :class:`PackedWeight`."""
    rows = x.rows if isinstance(x, ScaledRows) else x
    _gpu(rows, h, norm_weight)
    M, K = rows.shape
    N = w.shape[0]
    _need(rows.dtype == torch.bfloat16 and 0 < M <= 16, "gemm_skinny_residual takes bfloat16 x [M<=16, K] and w [N, K]")
    _need(K % 8 == 0 and rows.stride(1) == 1 and rows.stride(0) % 8 == 0 and rows.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    w_ptr, ldw = _weight_args(w, K, "gemm_skinny_residual")
    _need(h.dtype == torch.float32 and h.shape == (M, N) and h.stride(1) == 1, "h must be float32 [M, N]")
    _need(norm_weight.shape == (N,) and norm_weight.is_contiguous()
          and norm_weight.dtype in (torch.float32, torch.bfloat16), "norm_weight must be [N], float32 or bfloat16")
    n_parts = -(-N // 16)
    x_out = torch.empty((M, N), dtype=torch.bfloat16, device=rows.device)
    ssq_out = torch.empty((M, n_parts), dtype=torch.float32, device=rows.device)
    sc = _row_scale_args(x, M)
    st = _lib.load("gemm_skinny").fg_gemm_skinny_fused(
        _ptr(rows), rows.stride(0), w_ptr, ldw, ctypes.c_void_p(0), 0, M, N, K, 3, *sc,
        _ptr(h), h.stride(0), _ptr(norm_weight), _code(norm_weight), _ptr(x_out), x_out.stride(0), _ptr(ssq_out),
        _stream(rows))
    _check(st, "gemm_skinny_residual")
    return ScaledRows(x_out, ssq_out, N, float(eps))


def gemm_skinny(x, w, out_dtype: Optional[torch.dtype] = None,
                silu_mul_epilogue: bool = False, k_splits: int = 1, wide: Optional[bool] = None) -> torch.Tensor:
    """``x @ w.T`` for at most 128 rows of bf16 ``x`` on the matrix cores, built to
    stream ``w [N, K]`` (a matrix or :class:`PackedWeight`) once.  ``x`` may be :class:`ScaledRows` (at most 16 rows, bfloat16 out): the
    result rows are scaled.  With ``silu_mul_epilogue`` ``w`` is a gate/up matrix
    ordered by :func:`interleave_gate_up` and the result is ``silu(gate) * up``
    ``[M, N/2]`` (``"gelu_tanh"`` in True's place: that activation in SiLU's).  With ``k_splits > 1`` the k range is cut over workgroups and the
    result is fp32 ``[k_splits, M, N]`` partial sums (for few output columns,
    where one workgroup per 64 columns would leave most of the GPU idle).
    ``wide`` picks the kernel for 17..128 rows (64 columns a workgroup, x shared
    through LDS; it takes fewer rows and ``ScaledRows`` too); default: by the number of rows."""
    scaled = x if isinstance(x, ScaledRows) else None
    if scaled is not None:
        x = scaled.rows
    _gpu(x)
    _need(x.dtype == torch.bfloat16 and x.dim() == 2, "gemm_skinny takes bfloat16 x [M, K]")
    M, K = x.shape
    N = w.shape[0]
    _need(0 < M <= SKINNY_MAX_ROWS, f"gemm_skinny takes 1..{SKINNY_MAX_ROWS} rows, got {M}")
    _need(K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    w_ptr, ldw = _weight_args(w, K, "gemm_skinny")
    out_dtype = out_dtype or torch.bfloat16
    if silu_mul_epilogue:
        _need(N % 16 == 0 and out_dtype == torch.bfloat16, "the gate/up epilogue needs N % 16 == 0 and bf16 output")
    wide = (M > 16 or k_splits > 1) if wide is None else wide
    _need(M <= 64 or wide, "more than 64 rows take the wide kernel")
    _need(k_splits >= 1 and (k_splits == 1 or (wide and not silu_mul_epilogue)), "k_splits needs the wide kernel")
    if k_splits > 1:
        out_dtype = torch.float32
    cols = N // 2 if silu_mul_epilogue else N
    y = torch.empty((k_splits, M, cols) if k_splits > 1 else (M, cols), dtype=out_dtype, device=x.device)
    lib = _lib.load("gemm_skinny")
    if scaled is not None and wide:
        _need(M <= 16 and k_splits == 1 and out_dtype == torch.bfloat16, "scaled rows: at most 16 rows, bfloat16 out")
        st = lib.fg_gemm_skinny64(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), cols, ctypes.c_longlong(M * cols), 1, M, N,
            K, _code(y), _gated_code(silu_mul_epilogue), *_row_scale_args(scaled, M), _stream(x))
    elif scaled is not None:
        _need(M <= 16 and out_dtype == torch.bfloat16, "scaled rows: at most 16 rows, bfloat16 out")
        st = lib.fg_gemm_skinny_fused(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), y.stride(0), M, N, K, _gated_code(silu_mul_epilogue),
            *_row_scale_args(scaled, M), ctypes.c_void_p(0), 0, ctypes.c_void_p(0), 0, ctypes.c_void_p(0), 0,
            ctypes.c_void_p(0), _stream(x))
    elif wide:
        st = lib.fg_gemm_skinny64(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), cols, ctypes.c_longlong(M * cols), k_splits, M, N,
            K, _code(y), _gated_code(silu_mul_epilogue), *_row_scale_args(None, M), _stream(x))
    else:
        st = lib.fg_gemm_skinny(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), y.stride(0), M, N, K, _code(y),
            _gated_code(silu_mul_epilogue), _stream(x))
    _check(st, "gemm_skinny")
    return y


TILED_TILE_ROWS = (128, 256)  # rows of x a workgroup of the tiled kernel takes (by 128 columns)


def gemm_tiled(x: torch.Tensor, w, out_dtype: Optional[torch.dtype] = None,
               silu_mul_epilogue: bool = False, k_splits: int = 1, tile_rows: int = 128) -> torch.Tensor:
    """``x @ w.T`` for many rows of bf16 ``x`` by the engine's tiled MFMA kernel (both operands through a
    ring of LDS stages), with the k range cut over workgroups if ``k_splits > 1``: the result is then
    fp32 ``[k_splits, M, N]`` partial sums.  ``tile_rows``: 128 or 256 rows of x a workgroup (by 128
    columns).  With ``silu_mul_epilogue`` as :func:`gemm_skinny`; ``w`` a matrix or :class:`PackedWeight`."""
    _gpu(x)
    _need(x.dtype == torch.bfloat16 and x.dim() == 2, "gemm_tiled takes bfloat16 x [M, K]")
    M, K = x.shape
    N = w.shape[0]
    _need(M > 0 and K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    w_ptr, ldw = _weight_args(w, K, "gemm_tiled")
    _need(tile_rows in TILED_TILE_ROWS, f"tile_rows must be one of {TILED_TILE_ROWS}")
    out_dtype = out_dtype or torch.bfloat16
    if silu_mul_epilogue:
        _need(N % 16 == 0 and out_dtype == torch.bfloat16 and k_splits == 1,
              "the gate/up epilogue needs N % 16 == 0, bf16 output and one split")
    _need(1 <= k_splits <= 65535, "k_splits must be 1..65535")
    if k_splits > 1:
        out_dtype = torch.float32
    cols = N // 2 if silu_mul_epilogue else N
    y = torch.empty((k_splits, M, cols) if k_splits > 1 else (M, cols), dtype=out_dtype, device=x.device)
    st = _lib.load("gemm_tiled").fg_gemm_tiled(
        _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), cols, ctypes.c_longlong(M * cols), k_splits, M, N, K,
        _code(y), _gated_code(silu_mul_epilogue), int(tile_rows), _stream(x))
    _check(st, "gemm_tiled")
    return y


def gemm_skinny_qkv(x, wqkv, table: Optional[torch.Tensor], slots: torch.Tensor,
                    k_pages: torch.Tensor, v_pages: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                    rotary_dim: int, value_from_key: bool = False, gate: bool = False) -> torch.Tensor:
    """The q, k, v projections of at most 16 rows with :func:`rope_kv_write` in
    the product's epilogue: returns the rotated queries ``[M, H*hd]``; the rotated
    keys and the values go straight into their cache pages.  ``x`` may be :class:`ScaledRows`, ``wqkv`` a
    matrix or :class:`PackedWeight`.  ``value_from_key``: ``wqkv`` has no v rows, a token's value is its
    key before the rotation.  ``gate``: ``wqkv`` ends with ``H*hd`` rows of an output gate, and the result
    is ``[M, 2*H*hd]``: the queries, then the sigmoid of the gate."""
    scaled = x if isinstance(x, ScaledRows) else None
    if scaled is not None:
        x = scaled.rows
    _gpu(x, table, slots, k_pages, v_pages)
    _need(x.dim() == 2 and k_pages.dim() == 4, "x [M, K], wqkv [N, K], k_pages [n, KV, P, hd]")
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16,
          "gemm_skinny_qkv takes bfloat16")
    w_ptr, ldw = _weight_args(wqkv, K, "gemm_skinny_qkv")
    gate_cols = n_heads * head_dim if gate else 0
    n_rows = (n_heads + (1 if value_from_key else 2) * n_kv) * head_dim + gate_cols
    _need(0 < M <= 16 and tuple(wqkv.shape) == (n_rows, K), f"x [M<=16, K], wqkv [{n_rows}, K]")
    _need(K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    _need(head_dim % 16 == 0, "head size must be a multiple of 16")
    page_size = k_pages.shape[2]
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.shape[1:] == (n_kv, page_size, head_dim)
          and v_pages.shape == (k_pages.shape[0], n_kv, head_dim, page_size), "pages do not fit the heads")
    _i32(slots, "slots", M)
    if rotary_dim:
        _need(table is not None and table.dtype == torch.float32 and table.is_contiguous()
              and table.shape == (M, rotary_dim // 2, 2), "table must be float32 [M, rotary_dim/2, 2]")
    q = torch.empty((M, n_heads * head_dim + gate_cols), dtype=torch.bfloat16, device=x.device)
    st = _lib.load("gemm_skinny").fg_gemm_skinny_qkv(
        _ptr(x), x.stride(0), w_ptr, ldw, _ptr(q), q.stride(0), M, K,
        _ptr(table if rotary_dim else None), _ptr(slots), _ptr(k_pages), _ptr(v_pages), n_heads, n_kv, head_dim,
        rotary_dim, page_size, int(value_from_key), gate_cols, *_row_scale_args(scaled, M), _stream(x))
    _check(st, "gemm_skinny_qkv")
    return q


# ------------------------------------------------------------------- sampling
def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           top_p: Optional[torch.Tensor] = None, seeds: Optional[torch.Tensor] = None,
           counters: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token id per row of fp32 ``logits [n, V]``: argmax where the row's
    temperature is 0 (or none is given), else a draw from
    ``softmax(logits / temperature)`` cut to the ``top_p`` nucleus, with the
    uniform number taken from ``(seeds[row], counters[row])``.
    ``fastgen/generate.py:887-896``, ``utils/sampling.py:6-31``.
    """
    _gpu(logits, temperature, top_p, seeds, counters, out)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1,
          "logits must be float32 [n, V]")
    n, V = logits.shape
    out = torch.empty((n,), dtype=torch.int32, device=logits.device) if out is None else out
    _i32(out, "out", n)
    for name, t in (("temperature", temperature), ("top_p", top_p)):
        if t is not None:
            _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n, f"{name} must be float32 [n]")
    for name, t in (("seeds", seeds), ("counters", counters)):
        if t is not None:
            _need(t.dtype == torch.int64 and t.is_contiguous() and t.numel() >= n, f"{name} must be int64 [n]")
    if temperature is not None:
        _need(seeds is not None and counters is not None, "sampling needs seeds and counters")
    st = _lib.load("sampling").fg_sample(
        _ptr(logits), logits.stride(0), n, V, _ptr(temperature), _ptr(top_p), _ptr(seeds), _ptr(counters),
        _ptr(out), _stream(logits))
    _check(st, "sample")
    return out


def logprob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """``log_softmax(logits)[row, tokens[row]]`` (``fastgen/generate.py:725-730``)."""
    _gpu(logits, tokens)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1,
          "logits must be float32 [n, V]")
    n, V = logits.shape
    _i32(tokens, "tokens", n)
    out = torch.empty((n,), dtype=torch.float32, device=logits.device)
    st = _lib.load("sampling").fg_logprob(_ptr(logits), logits.stride(0), n, V, _ptr(tokens), _ptr(out), _stream(logits))
    _check(st, "logprob")
    return out


# ------------------------------------------------------------- routed experts
MOE_TILE_ROWS = (16, 32, 64, 128, 256)  # rows of one expert that a tile of the matrix-core kernels holds (from 128: through LDS)


def moe_route(x: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], top: int,
              sigmoid_scores: bool = False, correction: Optional[torch.Tensor] = None, n_groups: int = 1,
              keep_groups: int = 1, weight_scale: float = 1.0, softmax_scores: bool = False, n_extra: int = 0):
    """Per row of ``x [T, dim]``: fp32 logits ``x router^T + bias`` (``router`` fp32 ``[E, dim]``), the
    ``top`` largest (ties: the lower expert), and the softmax over those.  Returns int32 ``[T, top]``
    experts and fp32 ``[T, top]`` weights, the largest logit first.

    With ``sigmoid_scores`` an expert's score is ``sigmoid(logit)``; the choice goes by the score plus
    ``correction`` (fp32 ``[E]`` or None) among the experts of the ``keep_groups`` best of ``n_groups`` equal
    groups of neighbours (a group ranks by the sum of its two largest choice scores; ties: the lower group);
    the weights are the chosen experts' scores, without the correction, divided by their sum (+ 1e-20)
    and multiplied by ``weight_scale``.  ``softmax_scores``: the same with the softmax of the logits over all
    experts as the scores.

    ``n_extra``: ``router`` has that many rows behind the experts'; their logits (without bias) take no part in
    the choice and are returned as a third result, fp32 ``[T, n_extra]`` (the gate of a shared expert, say)."""
    _gpu(x, router, bias, correction)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.data_ptr() % 16 == 0, "x must be [T, dim] with unit column stride")
    T, dim = x.shape
    E = router.shape[0] - int(n_extra)
    _need(n_extra >= 0 and E >= 1 and not (sigmoid_scores and softmax_scores), "n_extra rows behind at least one expert; one way of scoring")
    _need(router.dtype == torch.float32 and router.shape == (E + n_extra, dim) and router.is_contiguous(),
          "router must be contiguous float32 [E + n_extra, dim]")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (E,) and bias.is_contiguous(), "bias must be float32 [E]")
    _need(1 <= top <= E, f"top={top} must be between 1 and the {E} experts")
    choice = torch.empty((T, top), dtype=torch.int32, device=x.device)
    weight = torch.empty((T, top), dtype=torch.float32, device=x.device)
    _f32_vec(correction, E, "correction")
    scored = sigmoid_scores or softmax_scores
    _need(scored or (correction is None and n_groups == 1), "correction and groups go with sigmoid or softmax scores")
    extra = torch.empty((T, n_extra), dtype=torch.float32, device=x.device) if n_extra else None
    _need(n_groups >= 1 and E % n_groups == 0 and 1 <= keep_groups <= n_groups and top <= keep_groups * (E // n_groups),
          f"{n_groups} groups of which {keep_groups} stay do not fit {E} experts and top={top}")
    st = _lib.load("moe").fg_moe_route_mode(_ptr(x), x.stride(0), _code(x), _ptr(router), _ptr(bias), T, dim, E, top,
                                            _ptr(choice), _ptr(weight), 2 if softmax_scores else int(bool(sigmoid_scores)),
                                            _ptr(correction), int(n_groups), int(keep_groups),
                                            ctypes.c_float(weight_scale), int(n_extra), _ptr(extra), _stream(x))
    _check(st, "moe_route")
    return (choice, weight, extra) if n_extra else (choice, weight)


def moe_max_tiles(n_pairs: int, n_experts: int, tile_rows: int) -> int:
    """The most tiles of ``tile_rows`` rows that ``n_pairs`` rows spread over ``n_experts`` can make."""
    return min(n_pairs, n_pairs // tile_rows + n_experts)


def moe_sort(choice: torch.Tensor, n_experts: int, tile_rows: int):
    """The (row, choice) pairs of ``choice [T, top]`` in the order of their experts, cut into tiles of
    at most ``tile_rows`` rows of one expert, on the device.  Returns int32 ``sorted [T * top]`` (pair
    ``t * top + j`` at each sorted place) and int32 ``tiles [max_tiles, 4]``: (expert, first sorted
    place, rows, 0), rows = 0 for tiles that this step does not have."""
    _gpu(choice)
    _i32(choice, "choice")
    n_pairs = choice.numel()
    max_tiles = moe_max_tiles(n_pairs, n_experts, tile_rows)
    sorted_ = torch.empty((n_pairs,), dtype=torch.int32, device=choice.device)
    tiles = torch.empty((max_tiles, 4), dtype=torch.int32, device=choice.device)
    st = _lib.load("moe").fg_moe_sort(_ptr(choice), n_pairs, n_experts, tile_rows, max_tiles, _ptr(sorted_), _ptr(tiles),
                                      _stream(choice))
    _check(st, "moe_sort")
    return sorted_, tiles


def _moe_mfma_ok(x: torch.Tensor, *weights: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and all(w.shape[2] % 8 == 0 and w.data_ptr() % 16 == 0 for w in weights))


def moe_gate_up(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, sorted_: torch.Tensor, tiles: torch.Tensor,
                top: int, tile_rows: int, limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """``silu(x_t W_gate[e]^T) * (x_t W_up[e]^T)`` for every pair, in the sorted order: ``[T * top, hidden]``.
    With ``limit`` > 0 the activation is the limited one: ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``,
    ``g * sigmoid(alpha * g) * (u + 1)``.
    ``w_gate``, ``w_up``: ``[E, hidden, dim]`` of ``x``'s dtype.  bfloat16 with sizes in multiples of 8
    runs on the matrix cores; everything else the fp32-FMA kernel (tiles of 16 rows only)."""
    _gpu(x, w_gate, w_up, sorted_, tiles)
    _need(x.dim() == 2 and x.stride(1) == 1 and w_gate.dim() == 3 and w_gate.shape == w_up.shape
          and w_gate.shape[2] == x.shape[1] and w_gate.is_contiguous() and w_up.is_contiguous()
          and w_gate.dtype == x.dtype == w_up.dtype, "x [T, dim], w_gate and w_up contiguous [E, hidden, dim] of x's dtype")
    _i32(sorted_, "sorted", x.shape[0] * top)
    _i32(tiles, "tiles")
    _need(tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.data_ptr() % 16 == 0, "tiles must be [n, 4], 16-byte aligned")
    hidden, dim = w_gate.shape[1], w_gate.shape[2]
    mfma = _moe_mfma_ok(x, w_gate) and hidden % 8 == 0
    _need(tile_rows in MOE_TILE_ROWS and (mfma or tile_rows == 16), "tile_rows does not fit the kernel")
    act = torch.empty((sorted_.numel(), hidden), dtype=x.dtype, device=x.device)
    st = _lib.load("moe").fg_moe_gate_up_act(_ptr(x), x.stride(0), _ptr(w_gate), _ptr(w_up), dim, _ptr(sorted_), _ptr(tiles),
                                             tiles.shape[0], tile_rows, top, dim, hidden, _ptr(act), hidden, _code(x),
                                             int(mfma), ACT_LIMITED if limit > 0 else 0, ctypes.c_float(limit),
                                             ctypes.c_float(alpha), _stream(x))
    _check(st, "moe_gate_up")
    return act


def moe_down(act: torch.Tensor, w_down: torch.Tensor, sorted_: torch.Tensor, tiles: torch.Tensor,
             tile_rows: int) -> torch.Tensor:
    """``act_p W_down[e]^T`` for every pair as fp32 ``[T * top, dim]``, row = pair (not the sorted order).
    ``w_down``: ``[E, dim, hidden]`` of ``act``'s dtype."""
    _gpu(act, w_down, sorted_, tiles)
    _need(act.dim() == 2 and act.is_contiguous() and w_down.dim() == 3 and w_down.is_contiguous()
          and w_down.shape[2] == act.shape[1] and w_down.dtype == act.dtype,
          "act contiguous [pairs, hidden], w_down contiguous [E, dim, hidden] of act's dtype")
    _i32(sorted_, "sorted", act.shape[0])
    _i32(tiles, "tiles")
    _need(tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.data_ptr() % 16 == 0, "tiles must be [n, 4], 16-byte aligned")
    dim, hidden = w_down.shape[1], w_down.shape[2]
    mfma = _moe_mfma_ok(act, w_down)
    _need(tile_rows in MOE_TILE_ROWS and (mfma or tile_rows == 16), "tile_rows does not fit the kernel")
    y = torch.empty((act.shape[0], dim), dtype=torch.float32, device=act.device)
    st = _lib.load("moe").fg_moe_down(_ptr(act), hidden, _ptr(w_down), hidden, _ptr(sorted_), _ptr(tiles), tiles.shape[0],
                                      tile_rows, dim, hidden, _ptr(y), _code(act), int(mfma), _stream(act))
    _check(st, "moe_down")
    return y


def moe_combine(y: torch.Tensor, weight: torch.Tensor, plus: Optional[torch.Tensor] = None,
                plus_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 ``[1, T, dim]``: ``plus[t] + sum_j weight[t, j] * y[t * top + j]``, the weighted sum first, ``j``
    ascending.  ``plus``: ``[T, dim]`` rows of any supported dtype, fp32 ``[S, T, dim]`` partial sums (a
    product whose k range was cut; summed in order), or None.  ``plus_gate``: fp32 ``[T]`` (any stride): the rows
    of ``plus`` are multiplied by ``sigmoid(plus_gate[t])`` before they are added."""
    _gpu(y, weight, plus, plus_gate)
    if plus_gate is not None:
        _need(plus is not None and plus_gate.dtype == torch.float32 and plus_gate.dim() == 1
              and plus_gate.shape[0] == weight.shape[0] and plus_gate.stride(0) >= 1, "plus_gate must be float32 [T], with plus")
    T, top = weight.shape
    _need(y.dtype == torch.float32 and y.dim() == 2 and y.shape[0] == T * top and y.is_contiguous()
          and weight.dtype == torch.float32 and weight.is_contiguous(), "y float32 [T * top, dim], weight float32 [T, top]")
    dim = y.shape[1]
    ldp, n_plus, stride = 0, 0, 0
    if plus is not None and plus.dim() == 3:
        _need(plus.dtype == torch.float32 and plus.shape[1:] == (T, dim) and plus.stride(2) == 1,
              "partial sums must be float32 [S, T, dim]")
        ldp, n_plus, stride = plus.stride(1), plus.shape[0], plus.stride(0)
    elif plus is not None:
        _need(plus.shape == (T, dim) and plus.stride(1) == 1, "plus must be [T, dim]")
        ldp, n_plus = plus.stride(0), 1
    out = torch.empty((1, T, dim), dtype=torch.float32, device=y.device)
    st = _lib.load("moe").fg_moe_combine_gated(_ptr(y), _ptr(weight), _ptr(plus), ldp, _code(plus) if plus is not None else F32,
                                               n_plus, ctypes.c_longlong(stride), T, top, dim, _ptr(out), _ptr(plus_gate),
                                               plus_gate.stride(0) if plus_gate is not None else 0, _stream(y))
    _check(st, "moe_combine")
    return out


# ------------------------------------------------------------- per-head work
class _PrepareArgs(ctypes.Structure):
    _fields_ = [("src", ctypes.c_void_p), ("src_stride", ctypes.c_int), ("bias", ctypes.c_void_p),
                ("n_q", ctypes.c_int), ("q_col", ctypes.c_int), ("q_w", ctypes.c_int), ("q_norm_dims", ctypes.c_int),
                ("q_norm_w", ctypes.c_void_p), ("q_out", ctypes.c_void_p), ("q_out_stride", ctypes.c_int),
                ("q_out_hw", ctypes.c_int), ("n_kv", ctypes.c_int), ("k_col", ctypes.c_int), ("k_w", ctypes.c_int),
                ("k_norm_dims", ctypes.c_int), ("k_norm_w", ctypes.c_void_p), ("v_col", ctypes.c_int),
                ("v_w", ctypes.c_int), ("table", ctypes.c_void_p), ("rot_start", ctypes.c_int),
                ("rotary_dim", ctypes.c_int), ("rot_q", ctypes.c_int), ("rot_k", ctypes.c_int), ("eps", ctypes.c_float), ("slots", ctypes.c_void_p),
                ("k_pages", ctypes.c_void_p), ("v_pages", ctypes.c_void_p), ("page_size", ctypes.c_int),
                ("hd_c", ctypes.c_int), ("norm_plain", ctypes.c_int), ("positions", ctypes.c_void_p),
                ("q_temp_coef", ctypes.c_float), ("q_temp_every", ctypes.c_int), ("v_first", ctypes.c_void_p),
                ("v_first_stride", ctypes.c_int), ("v_blend", ctypes.c_float)]


def _f32_vec(t: Optional[torch.Tensor], n: int, name: str) -> None:
    if t is not None:
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n, f"{name} must be contiguous float32 [{n}]")


def heads_prepare(src: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
                  n_q: int = 0, q_col: int = 0, q_width: int = 0, q_norm: Optional[torch.Tensor] = None,
                  q_norm_dims: int = 0, q_out: Optional[torch.Tensor] = None, q_out_width: int = 0,
                  n_kv: int = 0, k_col: int = 0, k_width: int = 0, k_norm: Optional[torch.Tensor] = None,
                  k_norm_dims: int = 0, v_col: int = -1, v_width: int = 0,
                  table: Optional[torch.Tensor] = None, rot_start: int = 0, rotary_dim: int = 0,
                  rotate_q: bool = True, rotate_k: bool = True, slots: Optional[torch.Tensor] = None, k_pages: Optional[torch.Tensor] = None,
                  v_pages: Optional[torch.Tensor] = None, norm_plain: bool = False,
                  positions: Optional[torch.Tensor] = None, q_temp_coef: float = 0.0, q_temp_every: int = 0,
                  v_first: Optional[torch.Tensor] = None, v_blend: float = 0.0) -> Optional[torch.Tensor]:
    """What lies between a product's rows ``src [T, width]`` (fp32, or the activation dtype) and an attention.

    Per token and head: add ``bias`` (fp32, per column of ``src``); RMS-norm the head's first ``*_norm_dims``
    elements with the fp32 weight ``*_norm`` (if given) and ``eps``; turn the pairs
    ``(rot_start + 2i, rot_start + 2i + 1)``, ``i < rotary_dim / 2``, by the angles of ``table``
    (:func:`rope_table`; ``rotate_q`` / ``rotate_k``: whether query and key heads turn).  The ``n_q`` query heads (``q_width`` wide, from column ``q_col``) go to
    ``q_out [T, n_q * q_out_width]`` of the cache's dtype, each padded with zeros to ``q_out_width``.
    The ``n_kv`` key heads (``k_width`` wide, from ``k_col``) go to ``slots`` of ``k_pages
    [n_pages, n_kv, P, hd]`` padded with zeros to ``hd``; the values (``v_width`` wide) to ``v_pages
    [n_pages, n_kv, hd, P]`` likewise: columns of their own from ``v_col``, with their bias, or, with
    ``v_col < 0``, the first ``v_width`` elements of the processed key.  A negative slot writes nothing.

    ``norm_plain``: heads with norm dimensions but no norm weight are divided by their root mean square.
    ``positions`` with ``q_temp_every > 0``: after its norm a query at position ``p`` is multiplied by
    ``1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1)``.  ``v_first [T, n_kv * v_width]`` (of ``src``'s
    dtype, unit column stride): the values become ``(1 - v_blend) v + v_blend v_first`` before they are stored."""
    _gpu(src, bias, q_norm, q_out, k_norm, table, slots, k_pages, v_pages, positions, v_first)
    _need(src.dim() == 2 and src.stride(1) == 1, "src must be [T, width] with unit column stride")
    T, width = src.shape
    a = _PrepareArgs()
    a.src, a.src_stride, a.bias, a.eps = src.data_ptr(), src.stride(0), bias.data_ptr() if bias is not None else None, eps
    _f32_vec(bias, width, "bias")
    act = None
    a.n_q, a.n_kv = int(n_q), int(n_kv)
    _need(n_q >= 0 and n_kv >= 0 and n_q + n_kv > 0, "there must be heads to prepare")
    if n_q:
        _need(q_out is not None and q_out.dim() == 2 and q_out.stride(1) == 1 and q_out.shape[0] == T
              and q_out.shape[1] >= n_q * q_out_width and q_out_width >= q_width > 0,
              "q_out must be [T, >= n_q * q_out_width] with q_out_width >= q_width")
        _need(q_col >= 0 and q_col + n_q * q_width <= width, "the query heads lie outside src")
        _need(q_width % 2 == 0 and q_out_width % 2 == 0 and q_out_width <= 1024, "head widths must be even, at most 1024")
        _need(0 <= q_norm_dims <= q_width and q_norm_dims % 2 == 0, "q_norm_dims must be even and at most q_width")
        _f32_vec(q_norm, q_norm_dims, "q_norm")
        _need(q_norm is None or q_norm_dims > 0, "a norm needs dimensions to run over")
        act = q_out.dtype
        a.q_col, a.q_w, a.q_norm_dims, a.q_norm_w = q_col, q_width, q_norm_dims, q_norm.data_ptr() if q_norm is not None else None
        a.q_out, a.q_out_stride, a.q_out_hw = q_out.data_ptr(), q_out.stride(0), q_out_width
    if n_kv:
        _need(slots is not None and k_pages is not None and v_pages is not None, "cache operands missing")
        _i32(slots, "slots", T)
        _need(k_pages.dim() == 4 and k_pages.is_contiguous() and k_pages.shape[1] == n_kv, "k_pages must be contiguous [n_pages, n_kv, P, hd]")
        n_pages, _, P, hd = k_pages.shape
        _need(v_pages.is_contiguous() and v_pages.shape == (n_pages, n_kv, hd, P) and v_pages.dtype == k_pages.dtype,
              "v_pages must be contiguous [n_pages, n_kv, hd, P] of k_pages' dtype")
        _need(act is None or act == k_pages.dtype, "q_out and the cache must share a dtype")
        act = k_pages.dtype
        _need(P % 8 == 0 and hd % 8 == 0 and hd <= 1024, "pages of a multiple of 8 tokens, head size a multiple of 8 up to 1024")
        _need(0 < k_width <= hd and k_width % 2 == 0 and 0 < v_width <= hd and v_width % 2 == 0,
              "key and value widths must be even and at most the cache's head size")
        _need(k_col >= 0 and k_col + n_kv * k_width <= width, "the key heads lie outside src")
        _need(v_col < 0 and v_width <= k_width or v_col >= 0 and v_col + n_kv * v_width <= width,
              "the values lie outside src (or, taken from the keys, are wider than they)")
        _need(0 <= k_norm_dims <= k_width and k_norm_dims % 2 == 0, "k_norm_dims must be even and at most k_width")
        _f32_vec(k_norm, k_norm_dims, "k_norm")
        _need(k_norm is None or k_norm_dims > 0, "a norm needs dimensions to run over")
        a.k_col, a.k_w, a.k_norm_dims, a.k_norm_w = k_col, k_width, k_norm_dims, k_norm.data_ptr() if k_norm is not None else None
        a.v_col, a.v_w = (v_col if v_col >= 0 else -1), v_width
        a.slots, a.k_pages, a.v_pages, a.page_size, a.hd_c = slots.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), P, hd
    if table is not None and rotary_dim:
        _need(table.dtype == torch.float32 and table.is_contiguous() and table.shape == (T, rotary_dim // 2, 2),
              "table must be float32 [T, rotary_dim/2, 2]")
        _need(rot_start >= 0 and rot_start % 2 == 0 and rotary_dim % 2 == 0, "the rotated run starts and ends at even dimensions")
        _need((not (n_q and rotate_q) or rot_start + rotary_dim <= q_width)
              and (not (n_kv and rotate_k) or rot_start + rotary_dim <= k_width), "the rotated run lies outside a head")
        a.table, a.rot_start, a.rotary_dim = table.data_ptr(), rot_start, rotary_dim
        a.rot_q, a.rot_k = int(bool(rotate_q)), int(bool(rotate_k))
    _need(src.dtype == torch.float32 or src.dtype == act, "src must be float32 or of the cache's dtype")
    a.norm_plain = int(bool(norm_plain))
    if positions is not None and q_temp_every > 0:
        _i32(positions, "positions", T)
        a.positions, a.q_temp_coef, a.q_temp_every = positions.data_ptr(), float(q_temp_coef), int(q_temp_every)
    if v_first is not None:
        _need(n_kv > 0 and v_col >= 0, "blended values need values of their own to blend")
        _need(v_first.dtype == src.dtype and v_first.dim() == 2 and v_first.stride(1) == 1 and v_first.shape[0] == T
              and v_first.shape[1] >= n_kv * v_width, "v_first must be [T, >= n_kv * v_width] of src's dtype")
        a.v_first, a.v_first_stride, a.v_blend = v_first.data_ptr(), v_first.stride(0), float(v_blend)
    st = _lib.load("heads").fg_heads_prepare(ctypes.byref(a), T, _code(src), _DTYPE_CODE[act], _stream(src))
    _check(st, "heads_prepare")
    return q_out


class _HeadLinearArgs(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("x_stride", ctypes.c_int), ("x_hs", ctypes.c_int), ("w", ctypes.c_void_p),
                ("y", ctypes.c_void_p), ("y_stride", ctypes.c_int), ("y_hs", ctypes.c_int), ("gate", ctypes.c_void_p),
                ("gate_stride", ctypes.c_int), ("T", ctypes.c_int), ("H", ctypes.c_int), ("N", ctypes.c_int),
                ("K", ctypes.c_int), ("tail", ctypes.c_int), ("y_hw", ctypes.c_int)]


def head_linear(x: torch.Tensor, x_head_stride: int, w: torch.Tensor, out: torch.Tensor, out_head_stride: int,
                tail: int = 0, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A product per head: ``out[t, h * out_head_stride + n] = sum_k w[h, n, k] * x[t, h * x_head_stride + k]``
    for ``w [H, N, K]``; with fp32 ``gate [T, >= H]`` (unit column stride) the result is multiplied by
    ``sigmoid(gate[t, h])``.  The ``tail`` columns of ``x``'s head behind ``K`` are copied behind the ``N``
    results, and what is left of the ``out_head_stride`` columns is set to zero."""
    _gpu(x, w, out, gate)
    _need(w.dim() == 3 and w.is_contiguous(), "w must be contiguous [H, N, K]")
    H, N, K = w.shape
    T = x.shape[0]
    _need(x.dim() == 2 and x.stride(1) == 1 and x_head_stride >= K + tail and x.shape[1] >= (H - 1) * x_head_stride + K + tail,
          "x must be [T, >= H * x_head_stride] with heads at least K + tail wide")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == T and out_head_stride >= N + tail
          and out.shape[1] >= H * out_head_stride, "out must be [T, >= H * out_head_stride] with heads at least N + tail wide")
    _need(x.dtype == w.dtype == out.dtype, "x, w and out must share a dtype")
    a = _HeadLinearArgs()
    a.x, a.x_stride, a.x_hs, a.w = x.data_ptr(), x.stride(0), x_head_stride, w.data_ptr()
    a.y, a.y_stride, a.y_hs = out.data_ptr(), out.stride(0), out_head_stride
    if gate is not None:
        _need(gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] == T and gate.shape[1] >= H
              and gate.dtype == torch.float32, "gate must be float32 [T, >= H]")
        a.gate, a.gate_stride = gate.data_ptr(), gate.stride(0)
    a.T, a.H, a.N, a.K, a.tail, a.y_hw = T, H, N, K, tail, out_head_stride
    mfma = (x.dtype == torch.bfloat16 and K % 8 == 0 and x.stride(0) % 8 == 0 and x_head_stride % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
    _need(mfma or K <= 1024, "heads of more than 1024 inputs need bfloat16 rows aligned to 16 bytes")
    st = _lib.load("heads").fg_head_linear(ctypes.byref(a), _code(x), int(mfma), _stream(x))
    _check(st, "head_linear")
    return out


def head_norm_gate(x: torch.Tensor, weight: torch.Tensor, eps: float, gate: torch.Tensor, n_heads: int,
                   out: torch.Tensor) -> torch.Tensor:
    """``out[t, h, :] = rmsnorm(x[t, h, :]) * weight * silu(gate[t, h, :])`` for fp32 ``x [T, H*e]``, fp32
    ``weight [e]`` shared by the heads, ``gate [T, >= H*e]`` (unit column stride) and ``out [T, H*e]`` of the
    activation dtype."""
    _gpu(x, weight, gate, out)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous() and x.shape[1] % n_heads == 0, "x must be contiguous float32 [T, H*e]")
    T, e = x.shape[0], x.shape[1] // n_heads
    _f32_vec(weight, e, "weight")
    _need(e <= 1024, "heads of at most 1024 elements")
    _need(out.shape == x.shape and out.is_contiguous(), "out must be contiguous [T, H*e]")
    _need(gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] == T and gate.shape[1] >= n_heads * e
          and gate.dtype == out.dtype, "gate must be [T, >= H*e] of out's dtype")
    st = _lib.load("heads").fg_head_norm_gate(_ptr(x), _ptr(weight), _ptr(gate), gate.stride(0), _ptr(out), T, n_heads,
                                              e, ctypes.c_float(eps), _code(out), _stream(out))
    _check(st, "head_norm_gate")
    return out


# ---------------------------------------------------------------- recurrence
def head_diff_norm(att: torch.Tensor, head_width: int, out: torch.Tensor, n_heads: int, group: int, v_width: int,
                   lam: float, eps: float, out_scale: float) -> torch.Tensor:
    """Two attention maps a head over one value: ``out[t, h, :] = n(a1 - lam * a2) * out_scale`` with ``n`` the
    division by the root mean square over the head's ``v_width`` values (``eps`` inside the root).  ``att [T, 2 H *
    head_width]`` holds, per key/value group of ``group`` query heads, the first maps' outputs of the group's heads
    and then the second maps' (each ``head_width`` wide, the first ``v_width`` columns count); ``out [T, H *
    v_width]`` of the same dtype."""
    _gpu(att, out)
    T = att.shape[0]
    _need(att.dim() == 2 and att.stride(1) == 1 and att.shape[1] >= 2 * n_heads * head_width and head_width >= v_width > 0,
          "att must be [T, >= 2 H * head_width] with heads at least v_width wide")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == T and out.shape[1] >= n_heads * v_width
          and out.dtype == att.dtype, "out must be [T, >= H * v_width] of att's dtype")
    _need(group >= 1 and n_heads % group == 0 and v_width <= 1024, "heads in whole groups, of at most 1024 values")
    st = _lib.load("heads").fg_head_diff_norm(_ptr(att), att.stride(0), head_width, _ptr(out), out.stride(0), T, n_heads,
                                              group, v_width, ctypes.c_float(lam), ctypes.c_float(eps),
                                              ctypes.c_float(out_scale), _code(att), _stream(att))
    _check(st, "head_diff_norm")
    return out


# ------------------------------------------------------- several residual streams
@dataclass
class StreamUpdate:
    """A sublayer's output on its way into several residual streams: ``rows`` (``[T, dim]`` of the activation
    dtype or fp32 ``[P, T, dim]`` partial sums) goes into stream ``t`` times ``out[t]`` while the streams are
    mixed by ``mix [S, S]`` (from-stream by to-stream): ``X'[t] = sum_s mix[s, t] X[s] + out[t] rows``.  What norms
    the streams next applies it (:func:`streams_step`)."""

    rows: torch.Tensor
    mix: torch.Tensor  # fp32 [S, S]
    out: torch.Tensor  # fp32 [S]


class _StreamArgs(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("delta", ctypes.c_void_p), ("parts", ctypes.c_void_p), ("n_parts", ctypes.c_int),
                ("part_stride", ctypes.c_longlong), ("mix", ctypes.c_void_p), ("out_w", ctypes.c_void_p),
                ("in_w", ctypes.c_void_p), ("norm_w", ctypes.c_void_p), ("out", ctypes.c_void_p), ("u_out", ctypes.c_void_p),
                ("rows", ctypes.c_void_p), ("n_streams", ctypes.c_int), ("n_tokens", ctypes.c_int), ("dim", ctypes.c_int),
                ("eps", ctypes.c_float)]


STREAMS_MAX = 16


def streams_spread(h: torch.Tensor, n_streams: int) -> torch.Tensor:
    """fp32 ``[S, T, dim]``: ``h [T, dim]`` copied into every one of ``n_streams`` residual streams."""
    _gpu(h)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous() and 1 <= n_streams <= STREAMS_MAX,
          f"h must be contiguous float32 [T, dim], at most {STREAMS_MAX} streams")
    x = torch.empty((n_streams, *h.shape), dtype=torch.float32, device=h.device)
    _check(_lib.load("streams").fg_streams_spread(_ptr(h), _ptr(x), ctypes.c_longlong(h.numel()), n_streams, _stream(h)),
           "streams_spread")
    return x


def streams_step(x: torch.Tensor, update: Optional[StreamUpdate], in_weights: Optional[torch.Tensor],
                 norm_weight: Optional[torch.Tensor], eps: float, out: Optional[torch.Tensor],
                 rows: Optional[torch.Tensor] = None, u_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """On the residual streams ``x`` (fp32 ``[S, T, dim]``), all in fp32: apply ``update`` (in place; None: nothing
    is pending), form ``u = sum_s in_weights[s] x[s]`` (``in_weights`` fp32 ``[S]``; None: the plain sum), and store
    ``out = rmsnorm(u) * norm_weight`` (``[T, dim]``, rounded once to its dtype; without ``norm_weight``: ``u`` itself)
    and/or ``u_out = u`` in fp32.  With ``rows`` only those tokens are computed, into consecutive rows, and ``x`` is
    left as it was."""
    _gpu(x, in_weights, norm_weight, out, rows, u_out, *(() if update is None else (update.rows, update.mix, update.out)))
    _need(x.dtype == torch.float32 and x.dim() == 3 and x.is_contiguous() and 1 <= x.shape[0] <= STREAMS_MAX,
          f"x must be contiguous float32 [S, T, dim], at most {STREAMS_MAX} streams")
    S, T, dim = x.shape
    _need(dim <= 8192, "rows of at most 8192 elements")
    n_rows = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, "rows")
    a = _StreamArgs()
    a.x, a.n_streams, a.n_tokens, a.dim, a.eps = x.data_ptr(), S, T, dim, eps
    act = out.dtype if out is not None else None
    if update is not None:
        _f32_vec(update.mix, S * S, "update.mix")
        _f32_vec(update.out, S, "update.out")
        _need(update.mix.numel() == S * S and update.out.numel() == S, "update.mix must be [S, S], update.out [S]")
        d = update.rows
        if d.dim() == 3:
            _need(d.dtype == torch.float32 and d.shape[1:] == (T, dim) and d.stride(2) == 1 and d.stride(1) == dim,
                  "partial sums must be float32 [P, T, dim] with contiguous rows")
            a.parts, a.n_parts, a.part_stride = d.data_ptr(), d.shape[0], d.stride(0)
        else:
            _need(d.shape == (T, dim) and d.is_contiguous() and (act is None or d.dtype == act),
                  "the update's rows must be contiguous [T, dim] of out's dtype")
            a.delta, act = d.data_ptr(), d.dtype
        a.mix, a.out_w = update.mix.data_ptr(), update.out.data_ptr()
    _need(update is not None or out is not None or u_out is not None, "nothing to apply and nothing to store")
    if in_weights is not None:
        _f32_vec(in_weights, S, "in_weights")
        a.in_w = in_weights.data_ptr()
    if norm_weight is not None:
        _need(norm_weight.shape == (dim,) and norm_weight.is_contiguous() and out is not None, "norm_weight must be [dim], with out")
        a.norm_w = norm_weight.data_ptr()
    if out is not None:
        _need(out.is_contiguous() and out.shape == (n_rows, dim), "out must be contiguous [rows, dim]")
        a.out = out.data_ptr()
    if u_out is not None:
        _need(u_out.is_contiguous() and u_out.shape == (n_rows, dim) and u_out.dtype == torch.float32,
              "u_out must be contiguous float32 [rows, dim]")
        a.u_out = u_out.data_ptr()
    if rows is not None:
        a.rows = rows.data_ptr()
    st = _lib.load("streams").fg_streams_step_rows(ctypes.byref(a), n_rows, _DTYPE_CODE[act or torch.float32],
                                                   _code(norm_weight) if norm_weight is not None else F32, _stream(x))
    _check(st, "streams_step")
    return out if out is not None else u_out


class _ScanArgs(ctypes.Structure):
    _fields_ = [("qkv", ctypes.c_void_p), ("row_stride", ctypes.c_int), ("q_col", ctypes.c_int), ("k_col", ctypes.c_int),
                ("v_col", ctypes.c_int), ("decay", ctypes.c_void_p), ("decay_stride", ctypes.c_int),
                ("q_scale", ctypes.c_float), ("state", ctypes.c_void_p),
                ("slot_ids", ctypes.c_void_p), ("q_start", ctypes.c_void_p), ("out", ctypes.c_void_p),
                ("H", ctypes.c_int), ("d", ctypes.c_int), ("e", ctypes.c_int), ("write_out", ctypes.c_int),
                ("write_state", ctypes.c_int)]


SCAN_CHUNK = 128  # tokens of a chunk where long runs of tokens are scanned chunk by chunk, side by side
SCAN_CHUNKED_FROM = 256  # the shortest run of tokens of one sequence for which a step is scanned so


def decay_scan(qkv: torch.Tensor, q_col: int, k_col: int, v_col: int, z: torch.Tensor, z_bias: Optional[torch.Tensor],
               tau: float, q_scale: float, state: torch.Tensor, slot_ids: torch.Tensor, q_start: torch.Tensor,
               n_seqs: int, out: torch.Tensor, q_start_host=None) -> torch.Tensor:
    """The recurrence ``S <- diag(a_t) S + k_t v_t^T``, ``o_t = S^T (q_t * q_scale)`` with
    ``a_t = sigmoid(z_t + z_bias)^(1/tau)``, token by token for every sequence of the step.

    ``qkv [T, width]`` holds per token ``q`` and ``k`` (``H*d`` columns from ``q_col`` / ``k_col``) and ``v``
    (``H*e`` from ``v_col``); ``z`` is fp32 ``[T, >= H*d]``; ``state`` fp32 ``[n_slots, H, d, e]`` is read at
    ``slot_ids[b]`` and left as the sequence's last token leaves it; sequence ``b`` has the tokens
    ``q_start[b] .. q_start[b+1]-1``; ``out`` is fp32 ``[T, H*e]``.

    ``q_start_host``: ``q_start`` on the host.  With it, a step in which a sequence brings ``SCAN_CHUNKED_FROM``
    tokens or more is scanned in chunks of ``SCAN_CHUNK`` tokens side by side (every chunk from a zero state,
    then the states that the chunks start from, then every chunk from its start); the result differs from
    the token-by-token scan's by rounding (a chunk's start state is summed in another order)."""
    _gpu(qkv, z, z_bias, state, slot_ids, q_start, out)
    _need(state.dtype == torch.float32 and state.dim() == 4 and state.is_contiguous(), "state must be contiguous float32 [n_slots, H, d, e]")
    _, H, d, e = state.shape
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and max(q_col, k_col) + H * d <= qkv.shape[1] and v_col + H * e <= qkv.shape[1]
          and min(q_col, k_col, v_col) >= 0, "q, k and v must lie inside the rows of qkv")
    _need(z.dtype == torch.float32 and z.dim() == 2 and z.stride(1) == 1 and z.shape[0] == T and z.shape[1] >= H * d,
          "z must be float32 [T, >= H*d]")
    _f32_vec(z_bias, H * d, "z_bias")
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, H * e), "out must be contiguous float32 [T, H*e]")
    _i32(slot_ids, "slot_ids", n_seqs)
    _i32(q_start, "q_start", n_seqs + 1)
    _need(d <= 512 and tau > 0, "at most 512 key channels a head; tau positive")
    a = _ScanArgs()
    a.qkv, a.row_stride, a.q_col, a.k_col, a.v_col = qkv.data_ptr(), qkv.stride(0), q_col, k_col, v_col
    # the decays of every token at once (exponentials and logarithms stay out of the chain of tokens)
    lib = _lib.load("recurrence")
    decay = torch.empty((T, H * d), dtype=torch.float32, device=z.device)
    st = lib.fg_decay_from_logits(_ptr(z), z.stride(0), _ptr(z_bias), ctypes.c_float(1.0 / tau), _ptr(decay), T, H * d,
                                  _stream(z))
    _check(st, "decay_from_logits")
    a.decay, a.decay_stride, a.q_scale, a.state = decay.data_ptr(), decay.stride(0), q_scale, state.data_ptr()
    a.slot_ids, a.q_start, a.out, a.H, a.d, a.e = slot_ids.data_ptr(), q_start.data_ptr(), out.data_ptr(), H, d, e
    a.write_out = a.write_state = 1
    lens = np.diff(np.asarray(q_start_host[: n_seqs + 1])) if q_start_host is not None else None
    if lens is None or not len(lens) or int(lens.max()) < SCAN_CHUNKED_FROM or torch.cuda.is_current_stream_capturing():
        st = lib.fg_decay_scan(ctypes.byref(a), int(n_seqs), _code(qkv), _stream(qkv))
        _check(st, "decay_scan")
        return out
    # chunk by chunk: the chunks' first tokens, and which chunks each sequence has
    starts, seq_chunk = [], [0]
    for b in range(n_seqs):
        starts.extend(range(int(q_start_host[b]), int(q_start_host[b + 1]), SCAN_CHUNK))
        seq_chunk.append(len(starts))
    n_chunks = len(starts)
    _need(n_chunks <= 65535 and n_seqs <= 65535, "too many chunks or sequences in one step")
    plan = upload(np.asarray(starts + [int(q_start_host[n_seqs])] + seq_chunk + list(range(n_chunks)), dtype=np.int32),
                  torch.int32, qkv.device)
    chunk_start, seq_chunk_d, chunk_ids = plan[: n_chunks + 1], plan[n_chunks + 1 : n_chunks + n_seqs + 2], plan[n_chunks + n_seqs + 2 :]
    chunks = torch.zeros((n_chunks, H, d, e), dtype=torch.float32, device=qkv.device)
    prod = torch.empty((n_chunks, H * d), dtype=torch.float32, device=qkv.device)
    _check(lib.fg_decay_chunk_product(_ptr(decay), decay.stride(0), _ptr(chunk_start), _ptr(prod), n_chunks, H * d,
                                      _stream(qkv)), "decay_chunk_product")
    a.state, a.slot_ids, a.q_start = chunks.data_ptr(), chunk_ids.data_ptr(), chunk_start.data_ptr()
    a.write_out, a.write_state = 0, 1  # what every chunk adds to a zero state
    _check(lib.fg_decay_scan(ctypes.byref(a), n_chunks, _code(qkv), _stream(qkv)), "decay_scan (chunks' sums)")
    _check(lib.fg_decay_chunk_states(_ptr(chunks), _ptr(prod), _ptr(state), _ptr(slot_ids), _ptr(seq_chunk_d), int(n_seqs),
                                     H, d, e, _stream(qkv)), "decay_chunk_states")
    a.write_out, a.write_state = 1, 0  # every chunk from the state it starts from
    _check(lib.fg_decay_scan(ctypes.byref(a), n_chunks, _code(qkv), _stream(qkv)), "decay_scan (chunks' outputs)")
    return out


# ----------------------------------------------------- gated activation, general
ACT_LIMITED = 3
_ACT_CODE = {"silu": 0, "gelu_tanh": 1, "relu": 2, "limited": ACT_LIMITED}


def gated_mul(gate_up: torch.Tensor, bias: Optional[torch.Tensor], activation: str, out_dtype: torch.dtype,
              out: Optional[torch.Tensor] = None, limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """``act(gate + b) * (up + b)`` for ``gate_up [T, 2 * hidden]`` as :func:`interleave_gate_up` orders it (fp32, or
    ``out_dtype``), ``bias`` fp32 ``[2 * hidden]`` in the same order (or None), ``activation`` one of ``silu``,
    ``gelu_tanh``, ``relu``, or ``limited``: ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``,
    ``g * sigmoid(alpha * g) * (u + 1)``.  All of it in fp32, one rounding to ``out_dtype``."""
    _gpu(gate_up, bias, out)
    _need(activation in _ACT_CODE, f"activation {activation!r} is not supported ({sorted(_ACT_CODE)})")
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 16 == 0,
          "gate_up must be contiguous [T, 2 * hidden], hidden a multiple of 8")
    T, hidden = gate_up.shape[0], gate_up.shape[1] // 2
    _need(gate_up.dtype == torch.float32 or gate_up.dtype == out_dtype, "gate_up must be float32 or of the result's dtype")
    _f32_vec(bias, 2 * hidden, "bias")
    if out is None:
        out = torch.empty((T, hidden), dtype=out_dtype, device=gate_up.device)
    _need(out.shape == (T, hidden) and out.is_contiguous() and out.dtype == out_dtype, "out must be contiguous [T, hidden]")
    _need(activation != "limited" or limit > 0, "the limited activation needs a positive limit")
    st = _lib.load("rows").fg_gated_mul_act(_ptr(gate_up), _ptr(bias), _ptr(out), T, hidden, _ACT_CODE[activation],
                                            ctypes.c_float(limit), ctypes.c_float(alpha), _code(gate_up), _code(out),
                                            _stream(out))
    _check(st, "gated_mul")
    return out


# ------------------------------------------------- selective state-space recurrence
class _SelectiveArgs(ctypes.Structure):
    _fields_ = [("u", ctypes.c_void_p), ("ldu", ctypes.c_int), ("dt", ctypes.c_void_p), ("lddt", ctypes.c_int),
                ("dt_bias", ctypes.c_void_p), ("A", ctypes.c_void_p), ("bc", ctypes.c_void_p), ("ldbc", ctypes.c_int),
                ("b_col", ctypes.c_int), ("c_col", ctypes.c_int), ("D", ctypes.c_void_p), ("z", ctypes.c_void_p),
                ("ldz", ctypes.c_int), ("x_raw", ctypes.c_void_p), ("ldx", ctypes.c_int), ("state", ctypes.c_void_p),
                ("row_len", ctypes.c_int), ("slot_ids", ctypes.c_void_p), ("q_start", ctypes.c_void_p),
                ("out", ctypes.c_void_p), ("ldo", ctypes.c_int), ("C", ctypes.c_int), ("N", ctypes.c_int),
                ("K", ctypes.c_int), ("LP", ctypes.c_int), ("write_out", ctypes.c_int), ("write_state", ctypes.c_int),
                ("write_tail", ctypes.c_int), ("dsum", ctypes.c_void_p)]


SELECTIVE_CHUNK = 32  # tokens of a chunk where long runs of tokens are scanned chunk by chunk, side by side
SELECTIVE_CHUNKED_FROM = 96  # the shortest run of tokens of one sequence for which a step is scanned so


def _rows_of_width(t: torch.Tensor, T: int, width: int, name: str) -> None:
    _need(t.dim() == 2 and t.stride(1) == 1 and t.shape[0] == T and t.shape[1] >= width,
          f"{name} must be [T, >= {width}] with unit column stride")


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, tail_off: int,
                slot_ids: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor, out: torch.Tensor,
                activation: Optional[str] = None) -> torch.Tensor:
    """A short causal convolution per channel over each sequence's tokens: ``out[t, c] = act(bias[c] + sum_j
    taps[c, j] x[t - (K - 1) + j, c])``, the last tap on the token itself.  ``x [T, >= C]``; ``taps`` fp32
    ``[C, K]``; tokens before this step's first are the last ``K - 1`` inputs of earlier steps, which
    ``state`` fp32 ``[n_slots, C, row_len]`` holds from column ``tail_off`` on at row ``slot_ids[seq]`` (zeros for
    a new request).  The state is read only (:func:`selective_scan` moves it on).  ``activation``: None or ``silu``."""
    _gpu(x, taps, bias, state, slot_ids, seq_of_token, q_start, out)
    C, K = taps.shape
    T = x.shape[0]
    _need(taps.dtype == torch.float32 and taps.is_contiguous(), "taps must be contiguous float32 [C, K]")
    _f32_vec(bias, C, "bias")
    _rows_of_width(x, T, C, "x")
    _rows_of_width(out, T, C, "out")
    _need(state.dtype == torch.float32 and state.dim() == 3 and state.is_contiguous() and state.shape[1] == C
          and 0 <= tail_off and tail_off + K - 1 <= state.shape[2], "state must be contiguous float32 [n_slots, C, >= tail_off + K - 1]")
    _need(activation in (None, "silu"), "activation must be None or 'silu'")
    _i32(seq_of_token, "seq_of_token", T)
    _i32(slot_ids, "slot_ids")
    _i32(q_start, "q_start")
    st = _lib.load("selective_scan").fg_causal_conv(
        _ptr(x), x.stride(0), _ptr(taps), _ptr(bias), _ptr(state), state.shape[2], int(tail_off), _ptr(slot_ids),
        _ptr(seq_of_token), _ptr(q_start), _ptr(out), out.stride(0), T, C, K, 1 if activation == "silu" else 0,
        _code(x), _code(out), _stream(out))
    _check(st, "causal_conv")
    return out


def selective_scan(u: torch.Tensor, dt: torch.Tensor, dt_bias: Optional[torch.Tensor], A: torch.Tensor, bc: torch.Tensor,
                   b_col: int, c_col: int, D: Optional[torch.Tensor], z: Optional[torch.Tensor],
                   x_raw: Optional[torch.Tensor], taps: int, state: torch.Tensor, slot_ids: torch.Tensor,
                   q_start: torch.Tensor, n_seqs: int, out: torch.Tensor, q_start_host=None) -> torch.Tensor:
    """The selective recurrence, token by token for every sequence of the step, in fp32:
    ``d = softplus(dt[t, c] + dt_bias[c])``; ``S[c, n] <- exp(d A[c, n]) S[c, n] + d u[t, c] B[t, n]``;
    ``out[t, c] = (sum_n S[c, n] C[t, n] + D[c] u[t, c]) * silu(z[t, c])``.

    ``u [T, >= C]`` and ``out`` have the activation dtype; ``dt [T, >= C]`` is fp32 or of the activation dtype; ``A``
    fp32 ``[C, N]``; ``B[t, n] = bc[t, b_col + n]``, ``C[t, n] = bc[t, c_col + n]``; ``state`` fp32 ``[n_slots, C,
    row_len]`` holds ``S`` in its first ``N`` columns and, behind them, the last ``taps - 1`` rows of ``x_raw`` (the
    input of the convolution that made ``u``), which this call moves on by the step's tokens.  Sequence ``b`` has
    the tokens ``q_start[b] .. q_start[b+1]-1`` and the state row ``slot_ids[b]``.

    ``q_start_host``: ``q_start`` on the host.  With it, a step in which a sequence brings ``SELECTIVE_CHUNKED_FROM``
    tokens or more is scanned in chunks of ``SELECTIVE_CHUNK`` tokens side by side (every chunk from a zero state,
    then the states that the chunks start from, then every chunk from its start); the result differs from the
    token-by-token scan's by rounding (a chunk's decay is the exponential of a sum, not a product)."""
    _gpu(u, dt, dt_bias, A, bc, D, z, x_raw, state, slot_ids, q_start, out)
    C, N = A.shape
    T = u.shape[0]
    act = out.dtype
    _need(A.dtype == torch.float32 and A.is_contiguous(), "A must be contiguous float32 [C, N]")
    _rows_of_width(u, T, C, "u")
    _rows_of_width(dt, T, C, "dt")
    _rows_of_width(out, T, C, "out")
    _need(u.dtype == act and bc.dtype == act and dt.dtype in (torch.float32, act), "u, bc and out share a dtype; dt is float32 or of it")
    _need(min(b_col, c_col) >= 0, "B and C must lie inside the rows of bc")
    _rows_of_width(bc, T, max(b_col, c_col) + N, "bc")
    _f32_vec(dt_bias, C, "dt_bias")
    _f32_vec(D, C, "D")
    a = _SelectiveArgs()
    if z is not None:
        _rows_of_width(z, T, C, "z")
        _need(z.dtype == act, "z must have out's dtype")
        a.z, a.ldz = z.data_ptr(), z.stride(0)
    _need(taps >= 1 and (taps == 1 or x_raw is not None), "the convolution's input is needed to move its tail on")
    if taps > 1:
        _rows_of_width(x_raw, T, C, "x_raw")
        _need(x_raw.dtype == act, "x_raw must have out's dtype")
        a.x_raw, a.ldx = x_raw.data_ptr(), x_raw.stride(0)
    _need(state.dtype == torch.float32 and state.dim() == 3 and state.is_contiguous() and state.shape[1] == C
          and state.shape[2] >= N + taps - 1, "state must be contiguous float32 [n_slots, C, >= N + taps - 1]")
    _i32(slot_ids, "slot_ids", n_seqs)
    _i32(q_start, "q_start", n_seqs + 1)
    spl = 4 if N <= 256 else 8 if N <= 512 else 16
    lanes = 1
    while lanes * spl < N:
        lanes *= 2
    _need(lanes <= 64, "at most 1024 states a channel")
    a.u, a.ldu, a.dt, a.lddt = u.data_ptr(), u.stride(0), dt.data_ptr(), dt.stride(0)
    a.dt_bias, a.A, a.D = (dt_bias.data_ptr() if dt_bias is not None else None), A.data_ptr(), (D.data_ptr() if D is not None else None)
    a.bc, a.ldbc, a.b_col, a.c_col = bc.data_ptr(), bc.stride(0), int(b_col), int(c_col)
    a.state, a.row_len, a.slot_ids, a.q_start = state.data_ptr(), state.shape[2], slot_ids.data_ptr(), q_start.data_ptr()
    a.out, a.ldo, a.C, a.N, a.K, a.LP = out.data_ptr(), out.stride(0), C, N, int(taps), lanes
    a.write_out = a.write_state = a.write_tail = 1
    lib = _lib.load("selective_scan")
    lens = np.diff(np.asarray(q_start_host[: n_seqs + 1])) if q_start_host is not None else None
    if lens is None or not len(lens) or int(lens.max()) < SELECTIVE_CHUNKED_FROM or torch.cuda.is_current_stream_capturing():
        _check(lib.fg_selective_scan(ctypes.byref(a), int(n_seqs), _code(dt), _code(out), _stream(out)), "selective_scan")
        return out
    # chunk by chunk: the chunks' first tokens, and which chunks each sequence has
    starts, seq_chunk = [], [0]
    for b in range(n_seqs):
        starts.extend(range(int(q_start_host[b]), int(q_start_host[b + 1]), SELECTIVE_CHUNK))
        seq_chunk.append(len(starts))
    n_chunks = len(starts)
    _need(n_chunks <= 65535 and n_seqs <= 65535, "too many chunks or sequences in one step")
    plan = upload(np.asarray(starts + [int(q_start_host[n_seqs])] + seq_chunk + list(range(n_chunks)), dtype=np.int32),
                  torch.int32, u.device)
    chunk_start, seq_chunk_d, chunk_ids = plan[: n_chunks + 1], plan[n_chunks + 1 : n_chunks + n_seqs + 2], plan[n_chunks + n_seqs + 2 :]
    row_len = state.shape[2]
    chunks = torch.zeros((n_chunks, C, row_len), dtype=torch.float32, device=u.device)
    dsum = torch.empty((n_chunks, C), dtype=torch.float32, device=u.device)
    a.state, a.slot_ids, a.q_start, a.dsum = chunks.data_ptr(), chunk_ids.data_ptr(), chunk_start.data_ptr(), dsum.data_ptr()
    a.write_out, a.write_state, a.write_tail = 0, 1, 0  # what every chunk adds to a zero state
    _check(lib.fg_selective_scan(ctypes.byref(a), n_chunks, _code(dt), _code(out), _stream(out)), "selective_scan (chunks' sums)")
    _check(lib.fg_scan_chunk_states(_ptr(chunks), _ptr(dsum), _ptr(A), _ptr(state), row_len, _ptr(slot_ids), _ptr(seq_chunk_d),
                                    _ptr(q_start), _ptr(x_raw), x_raw.stride(0) if x_raw is not None else 0, int(n_seqs), C, N,
                                    int(taps), _code(out), _stream(out)), "scan_chunk_states")
    a.write_out, a.write_state, a.dsum = 1, 0, None  # every chunk from the state it starts from
    _check(lib.fg_selective_scan(ctypes.byref(a), n_chunks, _code(dt), _code(out), _stream(out)), "selective_scan (chunks' outputs)")
    return out


# ----------------------------------------------------------- sigmoid attention
class _SigmoidAttentionArgs(ctypes.Structure):
    _fields_ = [("q", ctypes.c_void_p), ("q_stride", ctypes.c_int), ("q_hs", ctypes.c_int), ("k_pages", ctypes.c_void_p),
                ("v_pages", ctypes.c_void_p), ("block_table", ctypes.c_void_p), ("bt_stride", ctypes.c_int),
                ("seq_of_token", ctypes.c_void_p), ("positions", ctypes.c_void_p), ("n_tokens", ctypes.c_int),
                ("n_heads", ctypes.c_int), ("n_kv", ctypes.c_int), ("d", ctypes.c_int), ("e", ctypes.c_int),
                ("hd_c", ctypes.c_int), ("page_size", ctypes.c_int), ("scale", ctypes.c_float),
                ("dist_bias", ctypes.c_void_p), ("n_dist", ctypes.c_int), ("talk", ctypes.c_void_p),
                ("head_bias", ctypes.c_void_p), ("gate", ctypes.c_void_p), ("gate_stride", ctypes.c_int),
                ("out", ctypes.c_void_p), ("out_stride", ctypes.c_int), ("partial", ctypes.c_void_p),
                ("n_chunks", ctypes.c_int)]


def sigmoid_attention_chunk_keys() -> int:
    """Keys of one chunk: the sums over keys are kept per chunk and the chunks added in order."""
    return int(_lib.load("sigmoid_attention").fg_sigmoid_attention_chunk_keys())


class _SigmoidTileArgs(ctypes.Structure):
    _fields_ = [("q", ctypes.c_void_p), ("q_stride", ctypes.c_int), ("q_hs", ctypes.c_int), ("k_pages", ctypes.c_void_p),
                ("v_pages", ctypes.c_void_p), ("block_table", ctypes.c_void_p), ("bt_stride", ctypes.c_int),
                ("items", ctypes.c_void_p), ("n_items", ctypes.c_int), ("positions", ctypes.c_void_p),
                ("n_tokens", ctypes.c_int), ("n_heads", ctypes.c_int), ("n_kv", ctypes.c_int), ("d", ctypes.c_int),
                ("e", ctypes.c_int), ("page_size", ctypes.c_int), ("talk", ctypes.c_void_p), ("mixed", ctypes.c_void_p),
                ("n_dist", ctypes.c_int), ("gate", ctypes.c_void_p), ("gate_stride", ctypes.c_int), ("out", ctypes.c_void_p),
                ("out_stride", ctypes.c_int), ("partial", ctypes.c_void_p), ("n_chunks", ctypes.c_int),
                ("chunk_keys", ctypes.c_int)]


SIGMOID_TILE_TOKENS = 16  # query tokens of an item of the matrix-core kernel
SIGMOID_TILE_HEADS = 16  # the most heads it mixes
SIGMOID_TILE_CHUNK = 1024  # keys of a chunk, at least; at most SIGMOID_TILE_MAX_CHUNKS chunks
SIGMOID_TILE_MAX_CHUNKS = 8
SIGMOID_TILE_FEW_TOKENS = 64  # up to so many tokens a step, chunks of SIGMOID_TILE_FEW_CHUNK keys or more, as many as it takes
SIGMOID_TILE_FEW_CHUNK = 128


def sigmoid_attention_items(q_lens, q_start, n_cached) -> np.ndarray:
    """The step's sequences cut into items of up to 16 consecutive tokens: int32 ``[n, 4]`` of (sequence, first flat
    token, tokens, position of the first token), those with the most keys first."""
    items = [(b, int(q_start[b]) + i, min(SIGMOID_TILE_TOKENS, int(n) - i), int(n_cached[b]) + i)
             for b, n in enumerate(q_lens) for i in range(0, int(n), SIGMOID_TILE_TOKENS)]
    items.sort(key=lambda it: -(it[3] + it[2]))
    return np.asarray(items, dtype=np.int32).reshape(-1, 4)


def sigmoid_attention_mixed(scale: float, n_heads: int, dist_bias: Optional[torch.Tensor], talk: Optional[torch.Tensor],
                            head_bias: Optional[torch.Tensor], device):
    """What the matrix-core kernel takes in place of the table, the matrix and the biases (None with more than 16
    heads): the mixing matrix (or the identity) times the scale, zero padded to ``[16, 16]``, and ``[n_dist, 16]``:
    the distance table mixed over the heads by the same matrix plus the heads' biases (mixing is linear, so the
    bias can be mixed apart from the products and once for all steps).  fp32."""
    H = int(n_heads)
    if H > SIGMOID_TILE_HEADS:
        return None
    T = talk.float() if talk is not None else torch.eye(H, device=device)
    wide = torch.zeros((SIGMOID_TILE_HEADS, SIGMOID_TILE_HEADS), dtype=torch.float32, device=device)
    wide[:H, :H] = T * float(scale)
    rel = dist_bias.float() if dist_bias is not None else torch.zeros((1, H), device=device)
    m = rel @ T.T
    if head_bias is not None:
        m = m + head_bias.float()
    table = torch.zeros((m.shape[0], SIGMOID_TILE_HEADS), dtype=torch.float32, device=device)
    table[:, :H] = m
    return wide.contiguous(), table.contiguous()


def _sigmoid_attention_tiles(q, head_dim, out, v_head_dim, k_pages, v_pages, block_table, positions, n_heads, gate, max_keys,
                             items, mixed) -> torch.Tensor:
    T, H, d, e = q.shape[0], int(n_heads), int(head_dim), int(v_head_dim)
    _need(mixed is not None and len(mixed) == 2, "the matrix-core kernel takes sigmoid_attention_mixed's pair")
    talk, table = mixed
    _gpu(talk, table)
    _need(k_pages.dim() == 4 and k_pages.is_contiguous() and k_pages.dtype == torch.bfloat16, "k_pages must be contiguous bfloat16 [n_pages, G, P, hd]")
    n_pages, G, P, hd = k_pages.shape
    _need(v_pages.is_contiguous() and v_pages.shape == (n_pages, G, hd, P) and v_pages.dtype == torch.bfloat16,
          "v_pages must be contiguous bfloat16 [n_pages, G, hd, P]")
    _need(0 < H <= SIGMOID_TILE_HEADS and H % G == 0 and 0 < d <= hd and 0 < e <= hd and hd % 16 == 0 and hd <= 256 and P % 32 == 0,
          "at most 16 heads, head sizes at most the cache's (a multiple of 16 up to 256), pages of a multiple of 32 keys")
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "q and out must be bfloat16")
    _rows_of_width(q, T, H * d, "q")
    _rows_of_width(out, T, H * e, "out")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "block_table must be int32 [B, pages]")
    _i32(positions, "positions", T)
    _i32(items, "items")
    _need(items.dim() == 2 and items.shape[1] == 4 and items.is_contiguous() and items.data_ptr() % 16 == 0, "items must be [n, 4], 16-byte aligned")
    _need(talk.dtype == torch.float32 and talk.is_contiguous() and talk.shape == (SIGMOID_TILE_HEADS, SIGMOID_TILE_HEADS)
          and table.dtype == torch.float32 and table.is_contiguous() and table.dim() == 2 and table.shape[1] == SIGMOID_TILE_HEADS
          and table.data_ptr() % 16 == 0, "mixed must be sigmoid_attention_mixed's pair")
    a = _SigmoidTileArgs()
    if gate is not None:
        _need(gate.dtype == torch.float32 and gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] == T
              and gate.shape[1] >= H, "gate must be float32 [T, >= H]")
        a.gate, a.gate_stride = gate.data_ptr(), gate.stride(0)
    max_keys = max(int(max_keys), 1)
    if T <= SIGMOID_TILE_FEW_TOKENS:  # decoding: small chunks, so that few tokens give a workgroup for every compute unit
        chunk = min(SIGMOID_TILE_CHUNK, max(SIGMOID_TILE_FEW_CHUNK, -(-T * max_keys // (compute_units() * 32)) * 32))
    else:
        chunk = max(SIGMOID_TILE_CHUNK, -(-max_keys // (SIGMOID_TILE_MAX_CHUNKS * 32)) * 32)
    n_chunks = -(-max_keys // chunk)
    partial = None
    if n_chunks > 1:
        partial = torch.empty((n_chunks, T, H * e), dtype=torch.float32, device=q.device)
        a.partial = partial.data_ptr()
    a.n_chunks, a.chunk_keys = n_chunks, chunk
    a.q, a.q_stride, a.q_hs = q.data_ptr(), q.stride(0), d
    a.k_pages, a.v_pages, a.block_table, a.bt_stride = k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.stride(0)
    a.items, a.n_items, a.positions, a.n_tokens = items.data_ptr(), items.shape[0], positions.data_ptr(), T
    a.n_heads, a.n_kv, a.d, a.e, a.page_size = H, G, d, e, P
    a.talk, a.mixed, a.n_dist = talk.data_ptr(), table.data_ptr(), table.shape[0]
    a.out, a.out_stride = out.data_ptr(), out.stride(0)
    st = _lib.load(f"sigmoid_attention_mfma@{hd}").fg_sigmoid_attention_tiles(ctypes.byref(a), _stream(q))
    _check(st, "sigmoid_attention (matrix cores)")
    return out


def sigmoid_attention(q: torch.Tensor, head_dim: int, out: torch.Tensor, v_head_dim: int, k_pages: torch.Tensor,
                      v_pages: torch.Tensor, block_table: torch.Tensor, seq_of_token: torch.Tensor,
                      positions: torch.Tensor, n_heads: int, scale: float,
                      dist_bias: Optional[torch.Tensor] = None, talk: Optional[torch.Tensor] = None,
                      head_bias: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                      split_for: int = 0, items: Optional[torch.Tensor] = None, mixed=None) -> torch.Tensor:
    """Causal attention over the paged cache whose weights are sigmoids and are not normalised over the keys.

    For the query at flat row ``t`` (position ``p`` of sequence ``seq_of_token[t]``) and every key ``j <= p`` of its
    sequence: ``s_h = q_h . k_j * scale + dist_bias[min(p - j, n_dist - 1), h]``; the heads' scores are mixed,
    ``m_h = sum_g talk[h, g] s_g``; ``w_h = sigmoid(m_h + head_bias[h])``; ``out[t, h] = (sum_j w_h(j) v_j) *
    sigmoid(gate[t, h])``.  ``dist_bias`` fp32 ``[n_dist, H]``, ``talk`` fp32 ``[H, H]``, ``head_bias`` fp32 ``[H]`` and
    ``gate`` fp32 ``[T, >= H]`` may each be None.  ``q [T, >= H * head_dim]`` and ``out [T, >= H * v_head_dim]`` have
    the cache's dtype; keys and values are read from ``k_pages [n_pages, G, P, hd]`` and ``v_pages [n_pages, G, hd,
    P]`` (their first ``head_dim`` and ``v_head_dim`` elements).  ``split_for`` > 0: the keys of every token are
    cut over several workgroups, enough for sequences of that many keys (for few tokens with many keys); the
    result has the same bits either way.

    ``items`` (device int32 ``[n, 4]`` from :func:`sigmoid_attention_items`, covering every token of the step) and
    ``mixed`` (:func:`sigmoid_attention_mixed` of the same scale, table, matrix and biases): bfloat16 prompt portions
    on the matrix cores, an item a workgroup (``split_for``: the most keys a sequence has); the result differs from
    the general kernel's by rounding."""
    _gpu(q, out, k_pages, v_pages, block_table, seq_of_token, positions, dist_bias, talk, head_bias, gate, items)
    if items is not None:
        return _sigmoid_attention_tiles(q, head_dim, out, v_head_dim, k_pages, v_pages, block_table, positions, n_heads, gate,
                                        split_for, items, mixed)
    T, H, d, e = q.shape[0], int(n_heads), int(head_dim), int(v_head_dim)
    _need(k_pages.dim() == 4 and k_pages.is_contiguous(), "k_pages must be contiguous [n_pages, G, P, hd]")
    n_pages, G, P, hd = k_pages.shape
    _need(v_pages.is_contiguous() and v_pages.shape == (n_pages, G, hd, P) and v_pages.dtype == k_pages.dtype,
          "v_pages must be contiguous [n_pages, G, hd, P] of k_pages' dtype")
    _need(H > 0 and H % G == 0 and 0 < d <= hd and 0 < e <= hd and hd % 8 == 0 and P % 8 == 0,
          "heads must be a multiple of the cache's heads, head sizes at most the cache's")
    _need(q.dtype == k_pages.dtype and out.dtype == k_pages.dtype, "q and out must have the cache's dtype")
    _rows_of_width(q, T, H * d, "q")
    _rows_of_width(out, T, H * e, "out")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "block_table must be int32 [B, pages]")
    _i32(seq_of_token, "seq_of_token", T)
    _i32(positions, "positions", T)
    a = _SigmoidAttentionArgs()
    if dist_bias is not None:
        _need(dist_bias.dtype == torch.float32 and dist_bias.is_contiguous() and dist_bias.dim() == 2
              and dist_bias.shape[1] == H and dist_bias.shape[0] >= 1, "dist_bias must be contiguous float32 [n_dist, H]")
        a.dist_bias, a.n_dist = dist_bias.data_ptr(), dist_bias.shape[0]
    if talk is not None:
        _need(talk.dtype == torch.float32 and talk.is_contiguous() and talk.shape == (H, H), "talk must be contiguous float32 [H, H]")
        a.talk = talk.data_ptr()
    _f32_vec(head_bias, H, "head_bias")
    if head_bias is not None:
        a.head_bias = head_bias.data_ptr()
    if gate is not None:
        _need(gate.dtype == torch.float32 and gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] == T
              and gate.shape[1] >= H, "gate must be float32 [T, >= H]")
        a.gate, a.gate_stride = gate.data_ptr(), gate.stride(0)
    a.q, a.q_stride, a.q_hs = q.data_ptr(), q.stride(0), d
    a.k_pages, a.v_pages, a.block_table, a.bt_stride = k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.stride(0)
    a.seq_of_token, a.positions, a.n_tokens = seq_of_token.data_ptr(), positions.data_ptr(), T
    a.n_heads, a.n_kv, a.d, a.e, a.hd_c, a.page_size, a.scale = H, G, d, e, hd, P, float(scale)
    a.out, a.out_stride = out.data_ptr(), out.stride(0)
    partial = None
    if split_for > 0:
        n_chunks = -(-int(split_for) // sigmoid_attention_chunk_keys())
        if n_chunks > 1:
            partial = torch.empty((n_chunks, T, H * e), dtype=torch.float32, device=q.device)
            a.partial, a.n_chunks = partial.data_ptr(), n_chunks
    st = _lib.load("sigmoid_attention").fg_sigmoid_attention(ctypes.byref(a), _code(q), _stream(q))
    _check(st, "sigmoid_attention")
    return out
