"""Grouped causal attention whose weights are sigmoids: no softmax, no normalisation over the keys.

Per step: one product for q, k, v and a gate per head; q and k are divided by their root mean square per head (no
weight); a query at position ``p`` is multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``; keys and values
go to the pages.  The score of query ``i`` and key ``j <= i`` is ``q . k * scale + rel[bucket(i - j), h]`` (a learned
table per layer, one row a distance at first and logarithmic steps up to ``bias_far``, see
:func:`~fastgen_amd.parts.position.log_bucket`); the heads' scores of a pair are mixed by a matrix ``talk [H, H]``;
the weight is ``sigmoid(score + head_bias[h])``.  Each head's sum of weighted values is multiplied by the sigmoid
of its gate and projected.  Scores, mixing and weights are fp32 (``csrc/sigmoid_attention.hip``).

``value_mix``: the first such layer of a model keeps the values it computed for the step's tokens; every later one
stores ``(1 - lambda) v + lambda v_first`` in its cache, ``lambda`` a learned number of the layer.  (The layers find
each other through the step's context; the first one's ``lambda`` is not used.)

Options: ``dim``, ``n_heads``, ``n_kv_heads``, ``head_dim``, ``v_head_dim``, ``scale``, ``eps`` (of the unit norms),
``q_temp_coef``, ``q_temp_every`` (0: no temperature), ``bias_far`` and ``bias_rows`` (None: no distance bias),
``head_mix``, ``head_bias``, ``head_gate``, ``value_mix``, ``value_mix_stored``.
"""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, VECTOR, LayerStore, Mixer, PagedNeed, TensorSpec, place, register_part
from .position import distance_table

# so few tokens with so many keys that one workgroup a token would leave the device idle: the keys are cut
SPLIT_MAX_TOKENS = 64


class SigmoidAttention(Mixer):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.n_heads = int(o["n_heads"])
        self.n_kv_heads = int(o["n_kv_heads"])
        self.head_dim = int(o["head_dim"])
        self.v_head_dim = int(o.get("v_head_dim") or self.head_dim)
        self.scale = float(o.get("scale", self.head_dim ** -0.5))
        self.eps = float(o["eps"])
        self.q_temp_coef = float(o.get("q_temp_coef", 0.0))
        self.q_temp_every = int(o.get("q_temp_every", 0))
        self.bias_rows = int(o.get("bias_rows", 0))
        self.bias_far: Optional[float] = o.get("bias_far")
        self.head_mix = bool(o.get("head_mix", False))
        self.head_bias = bool(o.get("head_bias", False))
        self.head_gate = bool(o.get("head_gate", False))
        self.value_mix = bool(o.get("value_mix", False))
        # a layer that does not mix may still carry the number in its checkpoint: it is declared and not used
        self.value_mix_stored = self.value_mix or bool(o.get("value_mix_stored", False))
        if self.n_heads <= 0 or self.n_kv_heads <= 0 or self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.prefix}: n_heads={self.n_heads} is not a multiple of n_kv_heads={self.n_kv_heads}")
        if self.head_dim <= 0 or self.head_dim % 2 or self.v_head_dim <= 0 or self.v_head_dim % 2:
            raise ValueError(f"{self.prefix}: head sizes {self.head_dim} and {self.v_head_dim} must be positive and even")
        if self.q_temp_every < 0 or (self.bias_far is not None and self.bias_rows < 2):
            raise ValueError(f"{self.prefix}: q_temp_every must not be negative; a distance bias needs bias_rows")
        # a head in the cache: keys and values padded with zeros to one width, a multiple of 16
        self.cache_dim = -(-max(self.head_dim, self.v_head_dim) // 16) * 16
        if self.cache_dim > 512 or self.n_heads * self.v_head_dim > 4096 or self.n_heads > 64:
            raise ValueError(f"{self.prefix}: at most 64 heads of up to 512 dimensions, and 4096 value dimensions in all")
        self.w_in: Optional[StreamedMatrix] = None
        self.wo: Optional[StreamedMatrix] = None
        self.rel = self.talk = self.pb = None
        self.mixed = None  # what the matrix-core kernel takes in place of the table, the matrix and the biases
        self.blend = 0.0

    def tensor_specs(self) -> List[TensorSpec]:
        H, G, d, e = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim
        specs = [TensorSpec(self._name("q_proj.weight"), (H * d, self.dim)), TensorSpec(self._name("k_proj.weight"), (G * d, self.dim)),
                 TensorSpec(self._name("v_proj.weight"), (G * e, self.dim))]
        if self.bias_far is not None:
            specs.append(TensorSpec(self._name("distance_bias"), (self.bias_rows, H), VECTOR, ("normal", 0.5)))
        if self.value_mix_stored:
            specs.append(TensorSpec(self._name("value_mix"), (), VECTOR, ("normal", 0.3)))
        if self.head_mix:
            specs.append(TensorSpec(self._name("head_mix"), (H, H), VECTOR, ("normal", 0.3)))
        if self.head_bias:
            specs.append(TensorSpec(self._name("head_bias"), (H,), VECTOR, ("normal", 1.0)))
        if self.head_gate:
            specs.append(TensorSpec(self._name("gate_proj.weight"), (H, self.dim)))
        return specs + [TensorSpec(self._name("o_proj.weight"), (self.dim, H * e))]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        t = lambda name: tensors[self._name(name)]
        f32 = lambda name: t(name).to(device=device, dtype=torch.float32).contiguous()
        # one matrix for everything that reads the mixer's input: q, k, v, the heads' gates
        mats = [t("q_proj.weight"), t("k_proj.weight"), t("v_proj.weight")] + ([t("gate_proj.weight")] if self.head_gate else [])
        w = torch.cat(mats, dim=0)
        pad = -w.shape[0] % 8
        if pad:
            w = torch.cat([w, w.new_zeros(pad, self.dim)])
        self.w_in = streamed(place(w, MATRIX, dtype, device))
        self.wo = streamed(place(t("o_proj.weight"), MATRIX, dtype, device))
        if self.bias_far is not None:
            self.rel = distance_table(f32("distance_bias"), float(self.bias_far)).contiguous()
        if self.head_mix:
            self.talk = f32("head_mix")
        if self.head_bias:
            self.pb = f32("head_bias")
        if self.value_mix:
            self.blend = float(t("value_mix").float())
        self.mixed = ops.sigmoid_attention_mixed(self.scale, self.n_heads, self.rel, self.talk, self.pb, device)

    def paged_need(self) -> PagedNeed:
        return PagedNeed(self.n_kv_heads, self.cache_dim)

    def forward(self, x: torch.Tensor, ctx: Any, store: LayerStore) -> torch.Tensor:
        H, G, d, e = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim
        T = x.shape[0]
        group = ctx.groups[store.group]
        k_col, v_col, g_col = H * d, H * d + G * d, H * d + G * d + G * e
        rows = linear(x, self.w_in, out_dtype=torch.float32)  # fp32 [T, q | k | v | gates]
        v_first = None
        if self.value_mix:
            key = ("first_values", G, e)
            v_first = ctx.scratch.get(key)
            if v_first is None:
                ctx.scratch[key] = rows[:, v_col : v_col + G * e]
        q = torch.empty((T, H * d), dtype=x.dtype, device=x.device)
        ops.heads_prepare(
            rows, None, self.eps, n_q=H, q_col=0, q_width=d, q_norm_dims=d, q_out=q, q_out_width=d,
            n_kv=G, k_col=k_col, k_width=d, k_norm_dims=d, v_col=v_col, v_width=e,
            slots=group.slots, k_pages=store.k_pages, v_pages=store.v_pages, norm_plain=True,
            positions=ctx.positions, q_temp_coef=self.q_temp_coef, q_temp_every=self.q_temp_every,
            v_first=v_first, v_blend=self.blend)
        out = torch.empty((T, H * e), dtype=x.dtype, device=x.device)
        split_for, items = 0, None
        # bfloat16 with pages of a multiple of 32 keys and at most 16 heads: the matrix cores, an item of up to 16
        # tokens of a sequence a workgroup
        tiles_ok = (self.mixed is not None and x.dtype == torch.bfloat16 and store.k_pages.shape[2] % 32 == 0
                    and self.cache_dim <= 256)
        if tiles_ok and ctx.seq_records is not None and int(ctx.q_lens.max()) <= ops.SIGMOID_TILE_TOKENS:
            # every sequence is one item: its records are in the step's buffer already (and are refreshed with it
            # when the step is a replayed graph)
            items, split_for = ctx.seq_records, ctx.graph_capacity or ctx.max_kv_len
        elif T <= SPLIT_MAX_TOKENS:
            split_for = ctx.graph_capacity or ctx.max_kv_len
        elif tiles_ok and not ctx.graph_capacity:
            # prompt portions (if the step is not mostly single tokens, which would each be an item)
            items = ctx.scratch.get("sigmoid_items")
            if items is None:
                host = ops.sigmoid_attention_items(ctx.q_lens, ctx.q_start_host, ctx.n_cached)
                items = ctx.scratch["sigmoid_items"] = ops.upload(host, torch.int32, x.device) if 4 * len(host) <= T else False
            if items is False:
                items = None
            else:
                split_for = ctx.max_kv_len
        ops.sigmoid_attention(q, d, out, e, store.k_pages, store.v_pages, group.block_table, ctx.seq_of_token,
                              ctx.positions, H, self.scale, self.rel, self.talk, self.pb,
                              rows[:, g_col:] if self.head_gate else None, split_for=split_for, items=items, mixed=self.mixed)
        return linear(out, self.wo, partials_ok=True)


register_part("mixer", "sigmoid_attention", SigmoidAttention)
