"""Differential attention over the paged cache: every head has two score maps over one value.

A head's query and key come in two halves (``[map 1 | map 2]``, each ``head_dim`` wide); each half is an
attention of its own (own rotation, own softmax) over the head's values, and the head's output is

    o = a1 - lam * a2,   then o / sqrt(mean(o^2) + eps) * (1 - lambda_init)

with one number ``lam = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_init`` for the layer (four learned vectors of
``head_dim`` elements).  Heads are grouped (``n_kv_heads`` key/value heads).

How it runs: a map is a head of the engine's ordinary attention.  The layer keeps ``2 n_kv_heads`` key heads a
token in its pages (key/value group ``g``'s maps are heads ``2g`` and ``2g + 1``; the value is stored with both),
the query rows are ordered at load so that the heads that read key head ``2g + m`` lie together (per group: the
first maps of its heads, then the second maps), and the matrix-core attention kernels serve it as grouped
attention of ``2 n_heads`` heads; one small kernel then takes the difference and the norm per head
(``ops.head_diff_norm``).  Keys are cached after rotation; a layer with ``has_kv`` = False reads another layer's.

Options: ``dim``, ``n_heads``, ``n_kv_heads``, ``head_dim``, ``v_head_dim``, ``scale``, ``lambda_init``, ``eps``,
``position`` (a rotary scheme over a map of ``head_dim``), ``block`` (a token sees only the keys of its own block
of that many positions, counted from position 0; None: all before it), ``window`` (or a sliding one), ``has_kv``,
``exact_weights``.
"""

from __future__ import annotations

import math
from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, VECTOR, LayerStore, Mixer, PagedNeed, TensorSpec, build_part, place, register_part


class DifferentialAttention(Mixer):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.n_heads = int(o["n_heads"])
        self.n_kv_heads = int(o["n_kv_heads"])
        self.head_dim = int(o["head_dim"])
        self.v_head_dim = int(o.get("v_head_dim") or self.head_dim)
        self.scale = float(o.get("scale", self.head_dim ** -0.5))
        self.lambda_init = float(o["lambda_init"])
        self.eps = float(o["eps"])
        self.block: Optional[int] = o.get("block") or None
        self.window: Optional[int] = o.get("window") or None
        self.has_kv = bool(o.get("has_kv", True))
        self.exact_weights = bool(o.get("exact_weights", False))
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.prefix}: n_heads={self.n_heads} is not a multiple of n_kv_heads={self.n_kv_heads}")
        if self.block and self.window:
            raise ValueError(f"{self.prefix}: a mask of blocks and a sliding window do not go together")
        for name, v in (("head_dim", self.head_dim), ("v_head_dim", self.v_head_dim)):
            if v <= 0 or v % 2:
                raise ValueError(f"{self.prefix}: {name}={v} must be positive and even")
        # the width of a head in the cache: keys and values padded with zeros to one width, a multiple of 16
        self.cache_dim = -(-max(self.head_dim, self.v_head_dim) // 16) * 16
        if self.cache_dim > 512:
            raise ValueError(f"{self.prefix}: heads of {max(self.head_dim, self.v_head_dim)} are more than the attention kernels' 512")
        self.position = build_part("position", o["position"])
        self.w_in: Optional[StreamedMatrix] = None
        self.wo: Optional[StreamedMatrix] = None
        self.freqs: Optional[torch.Tensor] = None
        self.lam = 0.0

    @property
    def group(self) -> int:
        return self.n_heads // self.n_kv_heads

    def tensor_specs(self) -> List[TensorSpec]:
        H, G, d, e = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim
        specs = [TensorSpec(self._name("q_proj.weight"), (H * 2 * d, self.dim))]
        if self.has_kv:
            specs += [TensorSpec(self._name("k_proj.weight"), (G * 2 * d, self.dim)),
                      TensorSpec(self._name("v_proj.weight"), (G * e, self.dim))]
        specs += [TensorSpec(self._name(f"lambda_{n}"), (d,), VECTOR, ("normal", 0.1)) for n in ("q1", "k1", "q2", "k2")]
        return specs + [TensorSpec(self._name("o_proj.weight"), (self.dim, H * e))]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        H, G, d, e, D = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, self.dim
        t = lambda name: tensors[self._name(name)]
        # query rows [head, map, d] -> [group, map, head of the group, d]: the heads that read one key head lie together
        wq = t("q_proj.weight").view(G, self.group, 2, d, D).permute(0, 2, 1, 3, 4).reshape(H * 2 * d, D)
        mats = [self.position.arrange_rows(wq, 2 * H)]
        if self.has_kv:
            mats.append(self.position.arrange_rows(t("k_proj.weight"), 2 * G))
            # a group's value goes into the pages with both of its key heads
            mats.append(t("v_proj.weight").view(G, 1, e, D).expand(G, 2, e, D).reshape(2 * G * e, D))
        self.w_in = streamed(place(torch.cat(mats, dim=0), MATRIX, dtype, device))
        self.wo = streamed(place(t("o_proj.weight"), MATRIX, dtype, device))
        self.freqs = self.position.frequencies_on(device)
        f = lambda name: t(name).to(torch.float32)
        self.lam = (math.exp(float((f("lambda_q1") * f("lambda_k1")).sum()))
                    - math.exp(float((f("lambda_q2") * f("lambda_k2")).sum())) + self.lambda_init)

    def paged_need(self) -> PagedNeed:
        return PagedNeed(2 * self.n_kv_heads, self.cache_dim, self.window)

    def forward(self, x: torch.Tensor, ctx: Any, store: LayerStore) -> torch.Tensor:
        H, G, d, e, hc = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, self.cache_dim
        T = x.shape[0]
        group = ctx.groups[store.group]
        table = None
        if self.freqs is not None:
            key = ("rope_table", self.freqs.data_ptr())
            table = ctx.scratch.get(key)
            if table is None:
                table = ctx.scratch[key] = ops.rope_table(ctx.positions, self.freqs)
        writes = store.owns and self.has_kv
        q_width = 2 * H * d
        rows = linear(x, self.w_in if writes or not self.has_kv else self.w_in.first_rows(q_width), out_dtype=torch.float32)
        q = torch.empty((T, 2 * H * hc), dtype=x.dtype, device=x.device)
        ops.heads_prepare(
            rows, None, self.eps, n_q=2 * H, q_col=0, q_width=d, q_out=q, q_out_width=hc,
            n_kv=2 * G if writes else 0, k_col=q_width, k_width=d, v_col=q_width + 2 * G * d, v_width=e,
            table=table, rot_start=0, rotary_dim=self.position.rotary_dim,
            slots=group.slots if writes else None, k_pages=store.k_pages if writes else None,
            v_pages=store.v_pages if writes else None)
        att = torch.empty_like(q)
        ops.paged_attention(q, att, store.k_pages, store.v_pages, group, ctx, 2 * H, self.scale,
                            ops.block_mask(self.block) if self.block else (self.window or 0),
                            exact_weights=self.exact_weights)
        out = torch.empty((T, H * e), dtype=x.dtype, device=x.device)
        ops.head_diff_norm(att, hc, out, H, self.group, e, self.lam, self.eps, 1.0 - self.lambda_init)
        return linear(out, self.wo, partials_ok=True)


register_part("mixer", "differential_attention", DifferentialAttention)
