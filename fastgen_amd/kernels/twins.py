"""A plain PyTorch function beside every kernel of ``ops``: the same name, the
same arguments, the same effect on the same tensors, written as the formula
and not as the kernel works.  They say what each kernel computes and are what
the kernels are held to in ``tests/test_twins.py``; nothing of the engine
calls them (the engine has no execution path but its kernels), and they work
on CPU tensors as well as on GPU ones.

All arithmetic between a load and a store is fp32, as in the kernels; a result
is rounded once, to the dtype of the tensor it goes to.  Formulas:
``fastgen/forward.py:406-515``, ``fastgen/kernels/{rmsnorm,rope,paged_memcpy}.py``,
``fastgen/utils/sampling.py``.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.layout import store_k, store_v, unpack_k, unpack_v
from .ops import PackedWeight, PostNormed, ScaledRows  # noqa: F401


def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """``out[t] = table[tokens[t]] * scale`` as fp32."""
    out.copy_(table[tokens.long()].float() * scale)
    return out


def _added(delta: Optional[torch.Tensor]):
    """What a ``delta`` argument adds, in order: rows ``[T, dim]``, or fp32 partial sums ``[S, T, dim]``."""
    if delta is None:
        return []
    return [delta[s] for s in range(delta.shape[0])] if delta.dim() == 3 else [delta.float()]


def stream_add(h: torch.Tensor, delta: Optional[torch.Tensor], again: Optional[torch.Tensor],
               row: Optional[torch.Tensor]) -> torch.Tensor:
    """``h = ((h + delta) + again) + row`` in place, fp32, in that order; each term may be None."""
    for d in _added(delta):
        h += d
    if again is not None:
        h += again
    if row is not None:
        h += row[None, :]
    return h


def add_rows(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``a + b`` as fp32 ``[1, T, dim]``."""
    return (a.float() + b.float())[None]


def gate_mul(x: torch.Tensor, gate: torch.Tensor, sigmoid: bool = True) -> torch.Tensor:
    """``x *= sigmoid(gate)`` (or ``gate`` itself) over the first ``x.shape[1]`` columns of ``gate``, in place."""
    g = gate[:, : x.shape[1]].float()
    x.copy_((x.float() * (torch.sigmoid(g) if sigmoid else g)).to(x.dtype))
    return x


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h += delta`` (a ``[T, dim]`` tensor, or fp32 ``[S, T, dim]`` partial sums added in order), then
    ``out = h * rsqrt(mean(h^2) + eps) * weight``; with ``rows`` only those rows, and ``h`` stays as it was."""
    total = h.clone()
    if delta is not None and delta.dim() == 3:
        for s in range(delta.shape[0]):
            total += delta[s]
    elif delta is not None:
        total += delta.float()
    if rows is None:
        h.copy_(total)
    else:
        total = total[rows.long()]
    rstd = torch.rsqrt((total * total).sum(-1, keepdim=True) / total.shape[-1] + eps)
    out.copy_((total * rstd * weight.float()).to(out.dtype))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    xf = x.float()
    y = (xf * torch.rsqrt((xf * xf).sum(-1, keepdim=True) / x.shape[-1] + eps) * weight.float()).to(x.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of the gate and the up matrix in turns of 8: gate rows 8j..8j+7, then up rows 8j..8j+7."""
    F, K = gate.shape
    return torch.stack([gate.view(F // 8, 8, K), up.view(F // 8, 8, K)], dim=1).reshape(2 * F, K)


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` of ``[T, 2F]`` whose columns are interleaved in turns of 8 as above."""
    T, F2 = gate_up.shape
    gu = gate_up.float().view(T, F2 // 16, 2, 8)
    g, u = gu[:, :, 0].reshape(T, F2 // 2), gu[:, :, 1].reshape(T, F2 // 2)
    y = (g * torch.sigmoid(g) * u).to(gate_up.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def _gelu_tanh(g: torch.Tensor) -> torch.Tensor:
    return 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))


def _gated(y: torch.Tensor, epilogue) -> torch.Tensor:
    """``act(gate) * up`` of fp32 ``[M, 2F]`` interleaved in turns of 8; ``epilogue``: True or "silu", or "gelu_tanh"."""
    M, N = y.shape
    gu = y.view(M, N // 16, 2, 8)
    g, u = gu[:, :, 0].reshape(M, N // 2), gu[:, :, 1].reshape(M, N // 2)
    return (_gelu_tanh(g) if epilogue == "gelu_tanh" else g * torch.sigmoid(g)) * u


def gelu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``gelu_tanh(gate) * up`` of ``[T, 2F]`` whose columns are interleaved in turns of 8 as above."""
    y = _gated(gate_up.float(), "gelu_tanh").to(gate_up.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def post_add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], post_weight: Optional[torch.Tensor],
                     post_eps: float, weight: Optional[torch.Tensor], eps: float, out: Optional[torch.Tensor],
                     rows: Optional[torch.Tensor] = None, delta_bias: Optional[torch.Tensor] = None
                     ) -> Optional[torch.Tensor]:
    """``h += rmsnorm(delta + delta_bias) * post_weight`` (nothing without ``delta``); with ``weight``: ``out =
    rmsnorm(h) * weight``; with ``out`` alone: ``out = h``.  With ``rows`` only those rows, into consecutive rows of
    ``out``, and ``h`` stays."""
    s = h
    if delta is not None:
        d = sum(_added(delta))
        if delta_bias is not None:
            d = d + delta_bias.float()
        d = d * torch.rsqrt((d * d).mean(-1, keepdim=True) + post_eps) * post_weight.float()
        s = h + d
    if rows is None:
        h.copy_(s)
    else:
        s = s[rows.long()]
    if out is None:
        return out
    if weight is not None:
        s = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps) * weight.float()
    out.copy_(s.to(out.dtype))
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x = cap * tanh(x / cap)`` in place."""
    x.copy_(cap * torch.tanh(x / cap))
    return x


def scale_logits(x: torch.Tensor, factor: float) -> torch.Tensor:
    return x.mul_(factor)


def rope_table(positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """fp32 ``[T, len(freqs), 2]``: cos and sin of ``position * frequency``."""
    ang = positions.to(torch.float32)[:, None] * freqs.float()[None, :]
    return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1)


def _rotate(x: torch.Tensor, table: torch.Tensor, rotary_dim: int) -> torch.Tensor:
    """Interleaved pairs ``(2i, 2i+1)`` of the first ``rotary_dim`` head dims of ``x [T, heads, hd]`` (fp32)."""
    out = x.clone()
    if rotary_dim:
        cos, sin = table[:, None, :, 0], table[:, None, :, 1]
        a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        out[..., 0:rotary_dim:2] = a * cos - b * sin
        out[..., 1:rotary_dim:2] = b * cos + a * sin
    return out


def _write_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, slots: torch.Tensor, k: torch.Tensor,
                 v: torch.Tensor) -> None:
    """Rows ``k, v [T, KV, hd]`` into the pages at ``slots`` (page * P + offset; negative: not written)."""
    P = k_pages.shape[2]
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        page, off = divmod(s, P)
        for kvh in range(k_pages.shape[1]):
            store_k(k_pages, page, kvh, off, k[t, kvh].to(k_pages.dtype))
            store_v(v_pages, page, kvh, off, v[t, kvh].to(v_pages.dtype))


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, freqs: Optional[torch.Tensor], slots: torch.Tensor,
                  k_pages: torch.Tensor, v_pages: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                  rotary_dim: int, write_kv: bool = True, table: Optional[torch.Tensor] = None,
                  v_col: Optional[int] = None) -> torch.Tensor:
    """``qkv [T, >= H*hd (+ 2*KV*hd)]``: q is rotated in place; k is rotated and, with v, written into the
    pages (``fastgen/kernels/rope.py:56-89``, ``paged_memcpy.py:57-76``).  The values are the columns from
    ``v_col`` on (default: behind the keys; at the keys' own columns a value is its key before the rotation)."""
    T = qkv.shape[0]
    if rotary_dim and table is None:
        table = rope_table(positions, freqs)
    q_cols, kv_cols = n_heads * head_dim, n_kv * head_dim
    q = _rotate(qkv[:, :q_cols].float().view(T, n_heads, head_dim), table, rotary_dim)
    qkv[:, :q_cols] = q.reshape(T, q_cols).to(qkv.dtype)
    if write_kv:
        k = _rotate(qkv[:, q_cols : q_cols + kv_cols].float().view(T, n_kv, head_dim), table, rotary_dim)
        v_col = q_cols + kv_cols if v_col is None else v_col
        v = qkv[:, v_col : v_col + kv_cols].float().view(T, n_kv, head_dim)
        _write_pages(k_pages, v_pages, slots, k, v)
    return qkv


def _gather_kv(pages: torch.Tensor, unpack, table_row: torch.Tensor, n: int) -> torch.Tensor:
    """The first ``n`` keys (or values) of a sequence in natural order ``[n, KV, hd]``, fp32."""
    P = pages.shape[2] if unpack is unpack_k else pages.shape[3]
    natural = unpack(pages[table_row[: -(-n // P)].long()])  # [n_pages, KV, P, hd]
    return natural.permute(0, 2, 1, 3).reshape(-1, natural.shape[1], natural.shape[3])[:n].float()


def paged_attention_general(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                            block_table: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                            n_heads: int, scale: float, window: int = 0,
                            sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Token ``t`` of sequence ``b`` at position ``p`` attends keys ``0..p`` (``p-window+1..p`` with a window; with a
    negative one the keys up to ``p`` of its block of ``-window`` positions, blocks counted from 0)
    of its sequence, read through ``block_table[b]``; query head ``h`` reads kv head ``h // (H / KV)``;
    softmax of ``scale * q.k`` in fp32 (``fastgen/forward.py:176-258``).  With ``sinks`` head ``h``'s softmax runs
    over one more score, ``sinks[h]`` as it is, whose weight meets no value."""
    n_kv, P, hd = k_pages.shape[1], k_pages.shape[2], k_pages.shape[3]
    G = n_heads // n_kv
    for t in range(q.shape[0]):
        b, p = int(seq_of_token[t]), int(positions[t])
        k = _gather_kv(k_pages, unpack_k, block_table[b], p + 1)
        v = _gather_kv(v_pages, unpack_v, block_table[b], p + 1)
        lo = max(0, p - window + 1) if window > 0 else (p - p % -window if window < 0 else 0)
        qt = q[t, : n_heads * hd].float().view(n_heads, hd)
        for h in range(n_heads):
            s = (k[lo:, h // G] @ qt[h]) * scale
            if sinks is not None:
                s = torch.cat([s, sinks[h].float().reshape(1)])
            w = torch.softmax(s, 0)[: p + 1 - lo]
            out[t, h * hd : (h + 1) * hd] = (w @ v[lo:, h // G]).to(out.dtype)
    return out


def paged_attention_mfma(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                         block_table: torch.Tensor, small_items: Optional[torch.Tensor],
                         big_items: Optional[torch.Tensor], n_heads: int, scale: float, window: int = 0,
                         plan=None, max_chunks=None, min_tiles: int = 4, max_rows: int = 16,
                         tile_rows=None, exact_weights: bool = False,
                         sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same attention for tokens listed as items (sequence, first flat token, tokens, position of the
    first token).  How the kernels cut the work (``plan`` and what follows it) does not change the result;
    ``exact_weights`` only says how many digits of the softmax weights the kernel keeps (here: all)."""
    seq_of_token = torch.zeros(q.shape[0], dtype=torch.int32)
    positions = torch.zeros(q.shape[0], dtype=torch.int32)
    for items in (small_items, big_items):
        if items is None:
            continue
        for b, first, n, pos in items.reshape(-1, 4).tolist():
            seq_of_token[first : first + n] = b
            positions[first : first + n] = torch.arange(pos, pos + n, dtype=torch.int32)
    return paged_attention_general(q, out, k_pages, v_pages, block_table, seq_of_token, positions, n_heads, scale,
                                   window, sinks)


def paged_attention(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                    group, ctx, n_heads: int, scale: float, window: int = 0,
                    exact_weights: bool = False, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of one step: the block table from the layer's cache group, sequences and positions of the
    tokens from the step's context."""
    return paged_attention_general(q, out, k_pages, v_pages, group.block_table, ctx.seq_of_token, ctx.positions,
                                   n_heads, scale, window, sinks)


def gemm_nt(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
            out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x @ w.T`` with fp32 accumulation."""
    y = (x.float() @ w.float().T).to(out_dtype or (out.dtype if out is not None else x.dtype))
    if out is None:
        return y
    out.copy_(y)
    return out


def _rows(x) -> torch.Tensor:
    """The true rows of ``x``, a tensor or :class:`ScaledRows`, in fp32."""
    if isinstance(x, ScaledRows):
        return x.rows.float() * torch.rsqrt(x.ssq.sum(1, keepdim=True) / x.dim + x.eps)
    return x.float()


def _matrix(w) -> torch.Tensor:
    """The weight matrix ``[N, K]`` in fp32, from a matrix or from :class:`PackedWeight` (the inverse of the
    packing, written out: block ``[nb, ks]`` holds rows ``16 nb + r`` and k ``32 ks + 8 g + e`` at lane
    ``16 g + r``, element ``e``)."""
    if not isinstance(w, PackedWeight):
        return w.float()
    nb, ks = w.data.shape[:2]
    out = torch.zeros((nb * 16, ks * 32), dtype=torch.float32, device=w.data.device)
    for g in range(4):
        for r in range(16):
            out[r::16].view(nb, ks, 32)[:, :, 8 * g : 8 * g + 8] = w.data[:, :, 16 * g + r, :].float()
    return out[: w.n, : w.k]


def scale_rows(rows: torch.Tensor, ssq: torch.Tensor, dim: int, eps: float) -> torch.Tensor:
    return (rows.float() * torch.rsqrt(ssq.sum(1, keepdim=True) / dim + eps)).to(rows.dtype)


def gemm_skinny(x, w, out_dtype: Optional[torch.dtype] = None, silu_mul_epilogue: bool = False,
                k_splits: int = 1, wide: Optional[bool] = None) -> torch.Tensor:
    """``x @ w.T`` (``x`` may be :class:`ScaledRows`, ``w`` :class:`PackedWeight`: so in all three); with ``silu_mul_epilogue`` ``silu(gate) * up`` of a gate/up
    matrix interleaved in turns of 8; with ``k_splits > 1`` fp32 ``[S, M, N]`` partial sums over the k ranges
    ``[s * ceil(K / S / 256) * 256, ...)``.  ``wide`` only picks a kernel."""
    xf, wf = _rows(x), _matrix(w)
    if k_splits > 1:
        K = wf.shape[1]
        step = -(-K // (k_splits * 256)) * 256
        return torch.stack([xf[:, s * step : (s + 1) * step] @ wf[:, s * step : (s + 1) * step].T
                            for s in range(k_splits)])
    y = xf @ wf.T
    if silu_mul_epilogue:
        y = _gated(y, silu_mul_epilogue)
    return y.to(out_dtype or torch.bfloat16)


def gemm_tiled(x: torch.Tensor, w, out_dtype: Optional[torch.dtype] = None,
               silu_mul_epilogue: bool = False, k_splits: int = 1, tile_rows: int = 128) -> torch.Tensor:
    """``x @ w.T``; with ``silu_mul_epilogue`` as :func:`gemm_skinny`; with ``k_splits > 1`` fp32 ``[S, M, N]``
    partial sums over the k ranges ``[s * ceil(K / S / 32) * 32, ...)``.  ``tile_rows`` only picks a tile."""
    xf, wf = x.float(), _matrix(w)
    if k_splits > 1:
        K = wf.shape[1]
        step = -(-K // (k_splits * 32)) * 32
        return torch.stack([xf[:, s * step : (s + 1) * step] @ wf[:, s * step : (s + 1) * step].T
                            for s in range(k_splits)])
    y = xf @ wf.T
    if silu_mul_epilogue:
        y = _gated(y, silu_mul_epilogue)
    return y.to(out_dtype or torch.bfloat16)


def gemm_skinny_residual(x, w, h: torch.Tensor, norm_weight: torch.Tensor, eps: float) -> ScaledRows:
    """``h += x @ w.T``; returns what the RMSNorm after it needs: ``h * norm_weight`` in bfloat16 and the sums of
    squares of ``h`` over each block of 16 columns."""
    h += _rows(x) @ _matrix(w).T
    M, N = h.shape
    sq = torch.nn.functional.pad(h * h, (0, -N % 16)).view(M, -1, 16).sum(-1)
    return ScaledRows((h * norm_weight.float()).to(torch.bfloat16), sq, N, float(eps))


def gemm_skinny_qkv(x, wqkv, table: Optional[torch.Tensor], slots: torch.Tensor, k_pages: torch.Tensor,
                    v_pages: torch.Tensor, n_heads: int, n_kv: int, head_dim: int, rotary_dim: int,
                    value_from_key: bool = False, gate: bool = False) -> torch.Tensor:
    """The q, k, v projections with :func:`rope_kv_write` on the fp32 sums: returns the rotated queries in
    bfloat16; the rotated keys and the values go into the pages.  ``value_from_key``: there are no v rows,
    the values are the keys before the rotation.  ``gate``: ``H * hd`` more rows, whose sigmoid is returned
    behind the queries."""
    qkv = _rows(x) @ _matrix(wqkv).T
    T, q_cols, kv_cols = qkv.shape[0], n_heads * head_dim, n_kv * head_dim
    q = _rotate(qkv[:, :q_cols].view(T, n_heads, head_dim), table, rotary_dim)
    k_raw = qkv[:, q_cols : q_cols + kv_cols].view(T, n_kv, head_dim)
    k = _rotate(k_raw, table, rotary_dim)
    v_end = q_cols + kv_cols if value_from_key else q_cols + 2 * kv_cols
    v = k_raw if value_from_key else qkv[:, q_cols + kv_cols : v_end].view(T, n_kv, head_dim)
    _write_pages(k_pages, v_pages, slots, k, v)
    out = q.reshape(T, q_cols)
    if gate:
        out = torch.cat([out, torch.sigmoid(qkv[:, v_end : v_end + q_cols])], dim=1)
    return out.to(torch.bfloat16)


# ------------------------------------------------------------- routed experts
def moe_route(x: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], top: int,
              sigmoid_scores: bool = False, correction: Optional[torch.Tensor] = None, n_groups: int = 1,
              keep_groups: int = 1, weight_scale: float = 1.0, softmax_scores: bool = False, n_extra: int = 0):
    """The ``top`` experts with the largest fp32 logits ``x router^T + bias`` (largest first; of equal
    logits the lower expert) and the softmax over those logits alone.  With ``sigmoid_scores``: scores
    ``sigmoid(logit)``; chosen by score plus ``correction`` inside the ``keep_groups`` groups (of ``n_groups``) whose two
    largest choice scores sum highest; weights: the chosen scores over their sum (+ 1e-20), times ``weight_scale``.
    ``softmax_scores``: the same with scores ``softmax(logits)`` over all experts.  The last ``n_extra`` rows of
    ``router`` are no experts: their logits come back as a third result."""
    z = x.float() @ router.T
    E = router.shape[0] - n_extra
    z, extra = z[:, :E] + (bias if bias is not None else 0.0), z[:, E:]
    more = (extra,) if n_extra else ()
    if not (sigmoid_scores or softmax_scores):
        val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
        return (idx[:, :top].to(torch.int32), torch.softmax(val[:, :top], dim=-1), *more)
    score = torch.softmax(z, dim=-1) if softmax_scores else torch.sigmoid(z)
    choice = score + (correction if correction is not None else 0.0)
    T, E = choice.shape
    if n_groups > 1 and keep_groups < n_groups:
        per = E // n_groups
        rank = torch.sort(choice.view(T, n_groups, per), dim=-1, descending=True).values[..., : min(2, per)].sum(-1)
        order = torch.sort(rank, dim=-1, descending=True, stable=True).indices
        lost = torch.zeros(T, n_groups, dtype=torch.bool, device=x.device).scatter_(1, order[:, keep_groups:], True)
        choice = choice.masked_fill(lost[:, :, None].expand(T, n_groups, per).reshape(T, E), float("-inf"))
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    w = score.gather(1, idx)
    return (idx.to(torch.int32), w / (w.sum(-1, keepdim=True) + 1e-20) * weight_scale, *more)


def moe_max_tiles(n_pairs: int, n_experts: int, tile_rows: int) -> int:
    return min(n_pairs, n_pairs // tile_rows + n_experts)


def moe_sort(choice: torch.Tensor, n_experts: int, tile_rows: int):
    """The pairs (row, choice) in the order of their experts (within an expert in any order; here:
    ascending) and the tiles (expert, first sorted place, rows, 0) of at most ``tile_rows`` rows;
    tiles that do not exist have zero rows."""
    flat = choice.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    tiles = torch.zeros((moe_max_tiles(flat.numel(), n_experts, tile_rows), 4), dtype=torch.int32, device=choice.device)
    at, first = 0, 0
    for e, c in enumerate(torch.bincount(flat, minlength=n_experts).tolist()):
        for r in range(0, c, tile_rows):
            tiles[at] = torch.tensor([e, first + r, min(tile_rows, c - r), 0], dtype=torch.int32)
            at += 1
        first += c
    return order.to(torch.int32), tiles


def _expert_of_place(sorted_: torch.Tensor, tiles: torch.Tensor) -> torch.Tensor:
    expert = torch.zeros(sorted_.numel(), dtype=torch.long, device=sorted_.device)
    for e, first, rows, _ in tiles.tolist():
        expert[first : first + rows] = e
    return expert


def moe_gate_up(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, sorted_: torch.Tensor, tiles: torch.Tensor,
                top: int, tile_rows: int, limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """``silu(x_t w_gate[e]^T) * (x_t w_up[e]^T)`` for the pair at every sorted place, ``e`` its expert; with a
    ``limit``: ``g * sigmoid(alpha g) * (u + 1)`` of ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``."""
    expert = _expert_of_place(sorted_, tiles)
    rows = x[sorted_.long() // top].float()
    g = torch.einsum("pk,pfk->pf", rows, w_gate[expert].float())
    u = torch.einsum("pk,pfk->pf", rows, w_up[expert].float())
    return (_limited(g, u, limit, alpha) if limit > 0 else g * torch.sigmoid(g) * u).to(x.dtype)


def _limited(g: torch.Tensor, u: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    g, u = g.clamp(max=limit), u.clamp(min=-limit, max=limit)
    return g * torch.sigmoid(alpha * g) * (u + 1.0)


def moe_down(act: torch.Tensor, w_down: torch.Tensor, sorted_: torch.Tensor, tiles: torch.Tensor,
             tile_rows: int) -> torch.Tensor:
    """fp32 ``y[pair] = act[place of pair] w_down[e]^T``."""
    expert = _expert_of_place(sorted_, tiles)
    y = torch.empty((act.shape[0], w_down.shape[1]), dtype=torch.float32, device=act.device)
    y[sorted_.long()] = torch.einsum("pf,pdf->pd", act.float(), w_down[expert].float())
    return y


def moe_combine(y: torch.Tensor, weight: torch.Tensor, plus: Optional[torch.Tensor] = None,
                plus_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 ``[1, T, dim]``: ``plus[t] (* sigmoid(plus_gate[t])) + sum_j weight[t, j] * y[t * top + j]``."""
    T, top = weight.shape
    out = (weight[:, :, None] * y.view(T, top, -1)).sum(1)
    if plus is not None:
        p = plus.sum(0) if plus.dim() == 3 else plus.float()
        out = (p * torch.sigmoid(plus_gate.float())[:, None] if plus_gate is not None else p) + out
    return out[None]


def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           seeds: Optional[torch.Tensor] = None, counters: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy rows (no temperature, or temperature 0): the lowest index among the largest logits.  For rows with
    a temperature the kernel draws with a generator of its own keyed by (seed, counter); this function gives
    the set a draw must come from instead: -1 for such a row (see :func:`sample_support`)."""
    tok = torch.argmax(logits, dim=-1).to(torch.int32)  # torch.argmax returns the first of equal maxima
    if temperature is not None:
        tok = torch.where(temperature[: logits.shape[0]] > 0, torch.full_like(tok, -1), tok)
    if out is None:
        return tok
    out.copy_(tok)
    return out


def sample_support(logits: torch.Tensor, temperature: float, top_p: float) -> torch.Tensor:
    """bool ``[V]``: the tokens a draw with this temperature and nucleus can give, that is, those whose
    preceding mass in descending order of probability does not exceed ``top_p`` (``fastgen/utils/sampling.py:26-28``)."""
    probs = torch.softmax(logits.float() / temperature, -1)
    sort, idx = torch.sort(probs, descending=True)
    keep_sorted = ~(torch.cumsum(sort, -1) - sort > top_p)
    keep = torch.zeros_like(keep_sorted)
    keep[idx] = keep_sorted
    return keep


def logprob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """``log_softmax(logits)[row, tokens[row]]`` (``fastgen/generate.py:725-730``)."""
    return torch.log_softmax(logits.float(), -1)[torch.arange(logits.shape[0], device=logits.device), tokens.long()]


# ------------------------------------------------------------- per-head work
def heads_prepare(src: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
                  n_q: int = 0, q_col: int = 0, q_width: int = 0, q_norm: Optional[torch.Tensor] = None,
                  q_norm_dims: int = 0, q_out: Optional[torch.Tensor] = None, q_out_width: int = 0,
                  n_kv: int = 0, k_col: int = 0, k_width: int = 0, k_norm: Optional[torch.Tensor] = None,
                  k_norm_dims: int = 0, v_col: int = -1, v_width: int = 0,
                  table: Optional[torch.Tensor] = None, rot_start: int = 0, rotary_dim: int = 0,
                  rotate_q: bool = True, rotate_k: bool = True, slots: Optional[torch.Tensor] = None,
                  k_pages: Optional[torch.Tensor] = None, v_pages: Optional[torch.Tensor] = None, norm_plain: bool = False,
                  positions: Optional[torch.Tensor] = None, q_temp_coef: float = 0.0, q_temp_every: int = 0,
                  v_first: Optional[torch.Tensor] = None, v_blend: float = 0.0) -> Optional[torch.Tensor]:
    """Bias, a norm over the first dimensions of each head (``norm_plain``: also without a weight), the query's
    temperature ``1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1)``, the rotation of a run of pairs; queries to
    ``q_out`` and keys and values (blended with ``v_first``: ``(1 - v_blend) v + v_blend v_first``) to their pages,
    every head padded with zeros to its destination's width."""
    T = src.shape[0]
    x = src.float() + (bias.float()[None, : src.shape[1]] if bias is not None else 0.0)

    def heads(col, n, width, norm_w, norm_dims, turn, is_q=False):
        y = x[:, col : col + n * width].reshape(T, n, width).clone()
        if norm_w is not None or (norm_plain and norm_dims > 0):
            part = y[..., :norm_dims]
            part = part * torch.rsqrt((part * part).mean(-1, keepdim=True) + eps)
            y[..., :norm_dims] = part * norm_w.float()[:norm_dims] if norm_w is not None else part
        if is_q and positions is not None and q_temp_every > 0:
            steps = torch.div(positions.long() + 1, q_temp_every, rounding_mode="floor").float()
            y = y * (1.0 + q_temp_coef * torch.log(steps + 1.0))[:, None, None]
        if table is not None and rotary_dim and turn:
            run = y[..., rot_start : rot_start + rotary_dim]
            y[..., rot_start : rot_start + rotary_dim] = _rotate(run, table, rotary_dim)
        return y

    if n_q:
        q = heads(q_col, n_q, q_width, q_norm, q_norm_dims, rotate_q, True)
        wide = torch.zeros(T, n_q, q_out_width)
        wide[..., :q_width] = q.to(q_out.dtype).float().cpu()
        q_out[:, : n_q * q_out_width] = wide.reshape(T, -1).to(q_out.dtype).to(q_out.device)
    if n_kv:
        hd = k_pages.shape[3]
        k = heads(k_col, n_kv, k_width, k_norm, k_norm_dims, rotate_k)
        v = k[..., :v_width] if v_col < 0 else x[:, v_col : v_col + n_kv * v_width].reshape(T, n_kv, v_width)
        if v_first is not None:
            v = (1.0 - v_blend) * v + v_blend * v_first[:, : n_kv * v_width].float().reshape(T, n_kv, v_width)
        kw, vw = torch.zeros(T, n_kv, hd), torch.zeros(T, n_kv, hd)
        kw[..., :k_width], vw[..., :v_width] = k.cpu(), v.cpu()
        _write_pages(k_pages, v_pages, slots, kw, vw)
    return q_out


def head_linear(x: torch.Tensor, x_head_stride: int, w: torch.Tensor, out: torch.Tensor, out_head_stride: int,
                tail: int = 0, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t, h, :N] = w[h] @ x[t, h, :K]`` (times ``sigmoid(gate[t, h])``), then ``tail`` columns of ``x`` copied
    through, then zeros up to ``out_head_stride``."""
    H, N, K = w.shape
    T = x.shape[0]
    for h in range(H):
        xh = x[:, h * x_head_stride : h * x_head_stride + K + tail].float()
        y = xh[:, :K] @ w[h].float().T
        if gate is not None:
            y = y * torch.sigmoid(gate[:, h].float())[:, None]
        full = torch.zeros(T, out_head_stride, device=x.device)
        full[:, :N] = y
        full[:, N : N + tail] = xh[:, K:]
        out[:, h * out_head_stride : (h + 1) * out_head_stride] = full.to(out.dtype)
    return out


def head_norm_gate(x: torch.Tensor, weight: torch.Tensor, eps: float, gate: torch.Tensor, n_heads: int,
                   out: torch.Tensor) -> torch.Tensor:
    """RMS norm of every head of fp32 ``x [T, H*e]`` with one weight ``[e]``, times ``silu(gate)``."""
    T, e = x.shape[0], x.shape[1] // n_heads
    y = x.view(T, n_heads, e)
    y = y * torch.rsqrt((y * y).mean(-1, keepdim=True) + eps) * weight.float()
    g = gate[:, : n_heads * e].float().reshape(T, n_heads, e)
    out.copy_((y * g * torch.sigmoid(g)).reshape(T, -1).to(out.dtype))
    return out


def decay_scan(qkv: torch.Tensor, q_col: int, k_col: int, v_col: int, z: torch.Tensor, z_bias: Optional[torch.Tensor],
               tau: float, q_scale: float, state: torch.Tensor, slot_ids: torch.Tensor, q_start: torch.Tensor,
               n_seqs: int, out: torch.Tensor, q_start_host=None) -> torch.Tensor:
    """Per sequence and head, token by token: ``S = a[:, None] * S + k v^T``, ``o = S^T (q * q_scale)`` with
    ``a = sigmoid(z + z_bias) ** (1 / tau)``; ``S`` is the sequence's row of ``state``, updated in place.
    (``q_start_host`` only lets the kernels cut long runs of tokens into chunks.)"""
    _, H, d, e = state.shape
    for b in range(n_seqs):
        S = state[int(slot_ids[b])]
        for t in range(int(q_start[b]), int(q_start[b + 1])):
            row = qkv[t].float()
            q = row[q_col : q_col + H * d].view(H, d) * q_scale
            k = row[k_col : k_col + H * d].view(H, d)
            v = row[v_col : v_col + H * e].view(H, e)
            zt = z[t, : H * d].float() + (z_bias.float() if z_bias is not None else 0.0)
            a = torch.exp(torch.nn.functional.logsigmoid(zt) / tau).view(H, d)
            S.copy_(a[:, :, None] * S + k[:, :, None] * v[:, None, :])
            out[t] = torch.einsum("hde,hd->he", S, q).reshape(-1)
    return out


# ----------------------------------------------------- gated activation, general
def gated_mul(gate_up: torch.Tensor, bias: Optional[torch.Tensor], activation: str, out_dtype: torch.dtype,
              out: Optional[torch.Tensor] = None, limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """``act(gate + b) * (up + b)`` for rows interleaved in groups of 8 (gate, up); ``silu``, ``gelu_tanh``, ``relu``, or
    ``limited`` (``g * sigmoid(alpha g) * (u + 1)`` of the halves limited first)."""
    y = gate_up.float() + (bias.float() if bias is not None else 0.0)
    y = y.reshape(y.shape[0], -1, 2, 8)
    g, u = y[:, :, 0].reshape(y.shape[0], -1), y[:, :, 1].reshape(y.shape[0], -1)
    a = torch.relu(g) if activation == "relu" else _gelu_tanh(g) if activation == "gelu_tanh" else g * torch.sigmoid(g)
    r = (_limited(g, u, limit, alpha) if activation == "limited" else a * u).to(out_dtype)
    if out is None:
        return r
    out.copy_(r)
    return out


# ------------------------------------------------- selective state-space recurrence
def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, tail_off: int,
                slot_ids: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor, out: torch.Tensor,
                activation: Optional[str] = None) -> torch.Tensor:
    """Per sequence: the last ``K - 1`` inputs that the state holds, then this step's, convolved per channel."""
    C, K = taps.shape
    for b in range(q_start.numel() - 1):
        t0, t1 = int(q_start[b]), int(q_start[b + 1])
        if t1 <= t0:
            continue
        tail = state[int(slot_ids[b]), :, tail_off : tail_off + K - 1].T  # [K - 1, C], oldest first
        seq = torch.cat([tail.float(), x[t0:t1, :C].float()])
        y = sum(seq[j : j + t1 - t0] * taps[:, j].float() for j in range(K))
        if bias is not None:
            y = y + bias.float()
        if activation == "silu":
            y = y * torch.sigmoid(y)
        out[t0:t1, :C] = y.to(out.dtype)
    return out


def selective_scan(u: torch.Tensor, dt: torch.Tensor, dt_bias: Optional[torch.Tensor], A: torch.Tensor, bc: torch.Tensor,
                   b_col: int, c_col: int, D: Optional[torch.Tensor], z: Optional[torch.Tensor],
                   x_raw: Optional[torch.Tensor], taps: int, state: torch.Tensor, slot_ids: torch.Tensor,
                   q_start: torch.Tensor, n_seqs: int, out: torch.Tensor, q_start_host=None) -> torch.Tensor:
    """``S <- exp(d A) S + d u B``, ``y = S C + D u``, ``out = y * silu(z)`` token by token, ``d = softplus(dt + dt_bias)``; the
    state's rows hold ``S`` and behind it the convolution's last ``taps - 1`` inputs, moved on by this step.
    (``q_start_host`` only lets the kernels cut long runs of tokens into chunks.)"""
    C, N = A.shape
    for b in range(n_seqs):
        t0, t1 = int(q_start[b]), int(q_start[b + 1])
        row = state[int(slot_ids[b])]
        S = row[:, :N].clone()
        for t in range(t0, t1):
            d = torch.nn.functional.softplus(dt[t, :C].float() + (dt_bias if dt_bias is not None else 0.0))
            ut = u[t, :C].float()
            S = torch.exp(d[:, None] * A) * S + (d * ut)[:, None] * bc[t, b_col : b_col + N].float()[None, :]
            y = S @ bc[t, c_col : c_col + N].float() + (D * ut if D is not None else 0.0)
            if z is not None:
                zt = z[t, :C].float()
                y = y * zt * torch.sigmoid(zt)
            out[t, :C] = y.to(out.dtype)
        row[:, :N] = S
        if taps > 1 and t1 > t0:
            seq = torch.cat([row[:, N : N + taps - 1].T, x_raw[t0:t1, :C].float()])
            row[:, N : N + taps - 1] = seq[-(taps - 1):].T
    return out


# ----------------------------------------------------------- sigmoid attention
def sigmoid_attention(q: torch.Tensor, head_dim: int, out: torch.Tensor, v_head_dim: int, k_pages: torch.Tensor,
                      v_pages: torch.Tensor, block_table: torch.Tensor, seq_of_token: torch.Tensor,
                      positions: torch.Tensor, n_heads: int, scale: float,
                      dist_bias: Optional[torch.Tensor] = None, talk: Optional[torch.Tensor] = None,
                      head_bias: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                      split_for: int = 0, items: Optional[torch.Tensor] = None, mixed=None) -> torch.Tensor:
    """Token ``t`` at position ``p`` of sequence ``b`` over the keys ``0..p`` of its sequence: scores ``q . k * scale``
    plus ``dist_bias[min(p - j, n_dist - 1), h]``, mixed over the heads by ``talk``, plus ``head_bias``; weights
    ``sigmoid(score)``, not normalised; the heads' sums of weighted values times ``sigmoid(gate)``.  (``split_for``,
    ``items`` and ``mixed`` only choose how the kernels cut the work.)"""
    H, d, e = n_heads, head_dim, v_head_dim
    n_kv = k_pages.shape[1]
    rep = H // n_kv
    for t in range(q.shape[0]):
        b, p = int(seq_of_token[t]), int(positions[t])
        k = _gather_kv(k_pages, unpack_k, block_table[b], p + 1)[:, :, :d]
        v = _gather_kv(v_pages, unpack_v, block_table[b], p + 1)[:, :, :e]
        qt = q[t, : H * d].float().view(H, d)
        s = torch.einsum("hd,jhd->hj", qt, k.repeat_interleave(rep, dim=1)) * scale  # [H, p + 1]
        if dist_bias is not None:
            dist = (p - torch.arange(p + 1)).clamp(max=dist_bias.shape[0] - 1)
            s = s + dist_bias.float()[dist.to(dist_bias.device)].T
        if talk is not None:
            s = talk.float() @ s
        if head_bias is not None:
            s = s + head_bias.float()[:, None]
        o = torch.einsum("hj,jhe->he", torch.sigmoid(s), v.repeat_interleave(rep, dim=1))
        if gate is not None:
            o = o * torch.sigmoid(gate[t, :H].float())[:, None]
        out[t, : H * e] = o.reshape(-1).to(out.dtype)
    return out


# ------------------------------------------------------- two maps a head, several streams
def head_diff_norm(att: torch.Tensor, head_width: int, out: torch.Tensor, n_heads: int, group: int, v_width: int,
                   lam: float, eps: float, out_scale: float) -> torch.Tensor:
    """``out[t, h] = o / sqrt(mean(o^2) + eps) * out_scale`` with ``o = a1 - lam a2``; per key/value group ``att`` holds the
    first maps' outputs of the group's heads, then the second maps'."""
    T = att.shape[0]
    a = att[:, : 2 * n_heads * head_width].float().view(T, n_heads // group, 2, group, head_width)[..., :v_width]
    o = (a[:, :, 0] - lam * a[:, :, 1]).reshape(T, n_heads, v_width)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * out_scale
    out[:, : n_heads * v_width] = o.reshape(T, -1).to(out.dtype)
    return out


def streams_spread(h: torch.Tensor, n_streams: int) -> torch.Tensor:
    return h[None].repeat(n_streams, 1, 1)


def streams_step(x: torch.Tensor, update, in_weights: Optional[torch.Tensor], norm_weight: Optional[torch.Tensor],
                 eps: float, out: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                 u_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x' [t] = sum_s mix[s, t] x[s] + out_w[t] y`` (if an update is pending), ``u = sum_s in_weights[s] x'[s]``,
    ``out = rmsnorm(u) * norm_weight`` (or ``u``), ``u_out = u``; with ``rows`` only those tokens, ``x`` untouched."""
    S = x.shape[0]
    new = x
    if update is not None:
        y = update.rows.sum(0) if update.rows.dim() == 3 else update.rows.float()
        new = torch.einsum("sr,std->rtd", update.mix.view(S, S), x) + update.out.view(S, 1, 1) * y[None]
        if rows is None:
            x.copy_(new)
    u = new.sum(0) if in_weights is None else torch.einsum("s,std->td", in_weights, new)
    if rows is not None:
        u = u[rows.long()]
    if u_out is not None:
        u_out.copy_(u)
    if out is not None:
        n = u if norm_weight is None else u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * norm_weight.float()
        out.copy_(n.to(out.dtype))
    return out if out is not None else u_out
