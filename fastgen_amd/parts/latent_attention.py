"""Attention through latents: queries come from a narrow normed latent (or, without ``q_rank``, from one
projection of the mixer's input), keys and values from another one that is all the cache holds.

Per token the cache keeps one row for all heads: the normed key/value latent ``c`` (``kv_rank``
wide) followed by one rotated key part ``r`` (``rot_dim`` wide) that the heads share.  Head ``h``'s key
is ``[W_uk_h c ; r]`` and its value ``W_uv_h c``; neither is ever formed.  With
``q = [q_plain ; q_rot]`` the score is ``q_plain . (W_uk_h c) + q_rot . r = (W_uk_h^T q_plain) . c +
q_rot . r``: the query is carried into the latent's space (a product per head), attention runs
with one key/value head whose keys are the cached rows and whose values are their first
``kv_rank`` elements, and the heads' outputs, still in the latent's space, go through ``W_uv_h``
(a product per head again), times a sigmoid gate per head, into the output projection.

Options: ``dim``, ``n_heads``, ``head_dim`` (the plain part of a query or key), ``rot_dim``,
``v_head_dim``, ``kv_rank``, ``q_rank`` (None: no query latent; the tensor ``q_proj.weight`` gives the heads' queries
directly), ``scale``, ``window``, ``block`` (a mask of blocks of that many positions instead), ``sink``, ``head_gate``,
``eps`` (of the latents' norms), ``position`` (a rotary scheme over ``rot_dim`` dimensions).
"""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, VECTOR, LayerStore, Mixer, PagedNeed, TensorSpec, build_part, place, register_part


class LatentAttention(Mixer):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.n_heads = int(o["n_heads"])
        self.head_dim = int(o["head_dim"])
        self.rot_dim = int(o["rot_dim"])
        self.v_head_dim = int(o["v_head_dim"])
        self.kv_rank = int(o["kv_rank"])
        self.q_rank: Optional[int] = int(o["q_rank"]) if o.get("q_rank") else None
        self.scale = float(o.get("scale", (self.head_dim + self.rot_dim) ** -0.5))
        self.window: Optional[int] = o.get("window") or None
        self.block: Optional[int] = o.get("block") or None
        if self.block and self.window:
            raise ValueError(f"{self.prefix}: a mask of blocks and a sliding window do not go together")
        self.sink = bool(o.get("sink", False))
        self.head_gate = bool(o.get("head_gate", False))
        self.eps = float(o["eps"])
        self.exact_weights = bool(o.get("exact_weights", False))
        self.position = build_part("position", o["position"])
        if self.position.rotary_dim != self.rot_dim:
            raise ValueError(f"{self.prefix}: the rotary scheme turns {self.position.rotary_dim} dimensions, rot_dim is {self.rot_dim}")
        for name, v in (("head_dim", self.head_dim), ("rot_dim", self.rot_dim), ("kv_rank", self.kv_rank),
                        ("q_rank", self.q_rank or 2), ("v_head_dim", self.v_head_dim)):
            if v <= 0 or v % 2:
                raise ValueError(f"{self.prefix}: {name}={v} must be positive and even")
        # a cached row: the latent, the shared rotated part, zeros up to a multiple of 16
        self.cache_dim = -(-(self.kv_rank + self.rot_dim) // 16) * 16
        if self.cache_dim > 512:
            raise ValueError(f"{self.prefix}: kv_rank + rot_dim = {self.kv_rank + self.rot_dim} is more than the attention"
                             " kernels' head size of 512")
        self.w_in: Optional[StreamedMatrix] = None
        self.w_uq: Optional[StreamedMatrix] = None
        self.wo: Optional[StreamedMatrix] = None
        self.w_uk_t = self.w_uv = self.dq_norm = self.dkv_norm = self.sinks = self.freqs = None

    def tensor_specs(self) -> List[TensorSpec]:
        H, d, r, e, R, Q = self.n_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank, self.q_rank
        one = ("one_plus_normal", 0.01)
        if Q is None:
            specs = [TensorSpec(self._name("q_proj.weight"), (H * (d + r), self.dim))]
        else:
            specs = [TensorSpec(self._name("q_down.weight"), (Q, self.dim)),
                     TensorSpec(self._name("q_down_norm.weight"), (Q,), VECTOR, one),
                     TensorSpec(self._name("q_up.weight"), (H * (d + r), Q))]
        specs += [
            TensorSpec(self._name("kv_down.weight"), (R + r, self.dim)),
            TensorSpec(self._name("kv_down_norm.weight"), (R,), VECTOR, one),
            TensorSpec(self._name("k_up.weight"), (H * d, R)), TensorSpec(self._name("v_up.weight"), (H * e, R)),
        ]
        if self.sink:
            specs.append(TensorSpec(self._name("sinks"), (H,), VECTOR, ("normal", 1.0)))
        if self.head_gate:
            specs.append(TensorSpec(self._name("gate_proj.weight"), (H, self.dim)))
        return specs + [TensorSpec(self._name("o_proj.weight"), (self.dim, H * e))]

    def _interleave(self, w: torch.Tensor, heads: int, head_rows: int, start: int) -> torch.Tensor:
        """Rows ``start .. start + rot_dim`` of every head of ``w [heads * head_rows, in]`` from the checkpoint's
        pairing (``i`` with ``i + rot_dim/2``) to the kernels' (``2i`` with ``2i + 1``), if the scheme says so."""
        if getattr(self.position, "pairing", "interleaved") != "half":
            return w
        half = self.rot_dim // 2
        src = torch.arange(head_rows)
        src[start : start + self.rot_dim : 2] = start + torch.arange(half)
        src[start + 1 : start + self.rot_dim : 2] = start + half + torch.arange(half)
        full = (torch.arange(heads)[:, None] * head_rows + src[None, :]).reshape(-1)
        return w.index_select(0, full.to(w.device))

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        H, d, r, e, R = self.n_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank
        t = lambda name: tensors[self._name(name)]
        f32 = lambda name: t(name).to(device=device, dtype=torch.float32).contiguous()
        # one matrix for everything that reads the mixer's input: the query latent, the key/value latent with
        # the shared rotated part, the heads' gates
        # (without a query latent: the heads' queries themselves come first)
        first = t("q_down.weight") if self.q_rank else self._interleave(t("q_proj.weight"), H, d + r, d)
        mats = [first, self._interleave(t("kv_down.weight"), 1, R + r, R)]
        if self.head_gate:
            mats.append(t("gate_proj.weight"))
        self.w_in = streamed(place(torch.cat(mats, dim=0), MATRIX, dtype, device))
        if self.q_rank:
            self.w_uq = streamed(place(self._interleave(t("q_up.weight"), H, d + r, d), MATRIX, dtype, device))
        # per head: W_uk^T [R, d] carries a query into the latent's space, W_uv [e, R] a head's output out of it
        self.w_uk_t = place(t("k_up.weight").view(H, d, R).transpose(1, 2), MATRIX, dtype, device)
        self.w_uv = place(t("v_up.weight").view(H, e, R), MATRIX, dtype, device)
        self.wo = streamed(place(t("o_proj.weight"), MATRIX, dtype, device))
        self.dq_norm = f32("q_down_norm.weight") if self.q_rank else None
        self.dkv_norm = f32("kv_down_norm.weight")
        self.sinks = f32("sinks") if self.sink else None
        self.freqs = self.position.frequencies_on(device)

    def paged_need(self) -> PagedNeed:
        return PagedNeed(1, self.cache_dim, self.window)

    def forward(self, x: torch.Tensor, ctx: Any, store: LayerStore) -> torch.Tensor:
        H, d, r, e, R, Q, hc = (self.n_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank, self.q_rank,
                                self.cache_dim)
        T = x.shape[0]
        group = ctx.groups[store.group]
        key = ("rope_table", self.freqs.data_ptr())
        table = ctx.scratch.get(key)
        if table is None:
            table = ctx.scratch[key] = ops.rope_table(ctx.positions, self.freqs)
        rows = linear(x, self.w_in, out_dtype=torch.float32)  # [T, Q (or H (d + r)) | R + r | H] fp32
        own = store.owns
        if Q is None:
            Q = H * (d + r)  # the first columns are the heads' queries
            if own:
                ops.heads_prepare(
                    rows, None, self.eps, n_kv=1, k_col=Q, k_width=R + r, k_norm=self.dkv_norm, k_norm_dims=R, v_col=-1,
                    v_width=R, table=table, rot_start=R, rotary_dim=r, rotate_q=False, rotate_k=True, slots=group.slots,
                    k_pages=store.k_pages, v_pages=store.v_pages)
            q = torch.empty((T, Q), dtype=x.dtype, device=x.device)
            ops.heads_prepare(rows, None, self.eps, n_q=H, q_col=0, q_width=d + r, q_out=q, q_out_width=d + r,
                              table=table, rot_start=d, rotary_dim=r)
        else:
            cq = torch.empty((T, Q), dtype=x.dtype, device=x.device)
            ops.heads_prepare(
                rows, None, self.eps, n_q=1, q_col=0, q_width=Q, q_norm=self.dq_norm, q_norm_dims=Q, q_out=cq, q_out_width=Q,
                n_kv=1 if own else 0, k_col=Q, k_width=R + r, k_norm=self.dkv_norm, k_norm_dims=R, v_col=-1, v_width=R,
                table=table, rot_start=R, rotary_dim=r, rotate_q=False, rotate_k=True,
                slots=group.slots if own else None, k_pages=store.k_pages if own else None,
                v_pages=store.v_pages if own else None)
            q = linear(cq, self.w_uq)  # [T, H * (d + r)]
            ops.heads_prepare(q, None, self.eps, n_q=H, q_col=0, q_width=d + r, q_out=q, q_out_width=d + r,
                              table=table, rot_start=d, rotary_dim=r)
        q_lat = torch.empty((T, H * hc), dtype=x.dtype, device=x.device)
        ops.head_linear(q, d + r, self.w_uk_t, q_lat, hc, tail=r)
        lat = torch.empty_like(q_lat)
        ops.paged_attention(q_lat, lat, store.k_pages, store.v_pages, group, ctx, H, self.scale,
                            ops.block_mask(self.block) if self.block else (self.window or 0), exact_weights=self.exact_weights, sinks=self.sinks)
        out = torch.empty((T, H * e), dtype=x.dtype, device=x.device)
        ops.head_linear(lat, hc, self.w_uv, out, e, gate=rows[:, Q + R + r:] if self.head_gate else None)
        return linear(out, self.wo, partials_ok=True)


register_part("mixer", "latent_attention", LatentAttention)
