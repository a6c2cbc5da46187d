"""RMSNorm on the residual stream (``fastgen/kernels/rmsnorm.py:33-60``)."""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from .base import VECTOR, Norm, TensorSpec, place, register_part


class RMSNorm(Norm):
    """``y = x * rsqrt(mean(x^2) + eps) * weight`` in fp32, one rounding.  With the option
    ``unit_offset`` the checkpoint stores the weight around zero and ``1 + w`` is what multiplies
    (kept in fp32: the sum has more digits than bfloat16 holds)."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.dim = int(spec.options["dim"])
        self.eps = float(spec.options["eps"])
        self.unit_offset = bool(spec.options.get("unit_offset", False))
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        init = ("normal", 0.1) if self.unit_offset else ("one_plus_normal", 0.01)
        return [TensorSpec(self._name("weight"), (self.dim,), VECTOR, init)]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        w = tensors[self._name("weight")]
        self.weight = place(1.0 + w.to(torch.float32) if self.unit_offset else w, VECTOR, dtype, device)

    def fold_request(self, h: torch.Tensor):
        """(h, weight, eps): what a matrix product needs to fold the addition to the residual stream
        and this norm into its kernel (``fastgen_amd.kernels.linear.linear(residual=...)``)."""
        return (h, self.weight, self.eps)

    def forward(self, h, delta, dtype, rows=None):
        """``delta`` may be :class:`~fastgen_amd.kernels.ops.PostNormed`: a sublayer's output that is normed
        itself before it is added (the norm behind a sublayer); one kernel does that norm, the addition and
        this norm.  ``h`` may be several residual streams ``[S, T, dim]`` (``delta``: the
        :class:`~fastgen_amd.kernels.ops.StreamUpdate` still to be applied, or None): their sum is normed."""
        n = h.shape[-2] if rows is None else rows.numel()
        out = torch.empty((n, self.dim), dtype=dtype, device=h.device)
        if h.dim() == 3:
            return ops.streams_step(h, delta, None, self.weight, self.eps, out, rows)
        if isinstance(delta, ops.PostNormed):
            return ops.post_add_rmsnorm(h, delta.rows, delta.weight, delta.eps, self.weight, self.eps, out, rows,
                                        delta_bias=delta.bias)
        return ops.add_rmsnorm(h, delta, self.weight, self.eps, out, rows)


register_part("norm", "rmsnorm", RMSNorm)
