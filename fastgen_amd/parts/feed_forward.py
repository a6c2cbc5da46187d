"""Dense gated feed-forward (``fastgen/forward.py:483-499``):
``down(silu(gate(x)) * up(x))``.  Gate and up are one matrix with their rows
interleaved in groups of 8, so one product gives both and a tile of it holds
both halves of a channel: for few rows ``silu(gate) * up`` is applied where the
product is stored.  The option ``activation`` puts the tanh form of GELU
(``"gelu_tanh"``) or ReLU (``"relu"``) in SiLU's place, or the limited one (``"limited"`` with
``limit`` and ``alpha``: ``g * sigmoid(alpha g) * (u + 1)`` of ``g = min(gate, limit)``,
``u = clamp(up, -limit, limit)``).  With the option ``bias``
every projection has a bias: the gate's and the up projection's are added in
fp32 where the activation is applied to the product's fp32 result; the down
projection's (``output_bias``) is left to the kernel that adds the result to the
residual stream."""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, VECTOR, FeedForward, TensorSpec, place, register_part


class SwiGLU(FeedForward):
    folds_norms = True  # takes ScaledRows and the ``then`` request (see parts.block)

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.dim = int(spec.options["dim"])
        self.hidden_dim = int(spec.options["hidden_dim"])
        self.activation = spec.options.get("activation", "silu")
        if self.activation not in ("silu", "gelu_tanh", "relu", "limited"):
            raise ValueError(f"{self.prefix}: activation {self.activation!r} is not supported ('silu', 'gelu_tanh', 'relu',"
                             " 'limited')")
        self.limit, self.alpha = float(spec.options.get("limit") or 0.0), float(spec.options.get("alpha", 1.0))
        if (self.activation == "limited") != (self.limit > 0):
            raise ValueError(f"{self.prefix}: the limited activation, and only it, needs a positive limit")
        self.bias = bool(spec.options.get("bias", False))
        # the activation in a kernel of its own, on the product's rows: what the products' epilogues do not cover
        self.separate = self.bias or self.activation in ("relu", "limited")
        self.folds_norms = not self.separate
        self.b_gate_up: Optional[torch.Tensor] = None
        self.output_bias: Optional[torch.Tensor] = None
        self.w_gate_up: Optional[StreamedMatrix] = None
        self.w_down: Optional[StreamedMatrix] = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [
            TensorSpec(self._name("gate_proj.weight"), (self.hidden_dim, self.dim)),
            TensorSpec(self._name("up_proj.weight"), (self.hidden_dim, self.dim)),
            TensorSpec(self._name("down_proj.weight"), (self.dim, self.hidden_dim)),
        ]
        if self.bias:
            specs += [TensorSpec(self._name("gate_proj.bias"), (self.hidden_dim,), VECTOR, ("normal", 0.1)),
                      TensorSpec(self._name("up_proj.bias"), (self.hidden_dim,), VECTOR, ("normal", 0.1)),
                      TensorSpec(self._name("down_proj.bias"), (self.dim,), VECTOR, ("normal", 0.1))]
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        gate, up = tensors[self._name("gate_proj.weight")], tensors[self._name("up_proj.weight")]
        down = tensors[self._name("down_proj.weight")]
        pad = -self.hidden_dim % 8
        if pad:
            # the kernels work on groups of 8 channels: channels of zero weights are added, whose
            # activation silu(0) * 0 = 0 meets zero columns of the down projection
            gate = torch.cat([gate, gate.new_zeros(pad, self.dim)])
            up = torch.cat([up, up.new_zeros(pad, self.dim)])
            down = torch.cat([down, down.new_zeros(self.dim, pad)], dim=1)
        self.w_gate_up = streamed(place(ops.interleave_gate_up(gate, up), MATRIX, dtype, device))
        self.w_down = streamed(place(down, MATRIX, dtype, device))
        if self.bias:
            f32 = lambda name: tensors[self._name(name)].to(torch.float32)
            bg, bu = f32("gate_proj.bias"), f32("up_proj.bias")
            if pad:
                bg, bu = torch.cat([bg, bg.new_zeros(pad)]), torch.cat([bu, bu.new_zeros(pad)])
            # in the order of the interleaved matrix's rows
            self.b_gate_up = ops.interleave_gate_up(bg[:, None], bu[:, None])[:, 0].to(device=device).contiguous()
            self.output_bias = f32("down_proj.bias").to(device=device).contiguous()

    def forward(self, x, then=None):
        """``x``: the normed rows, or ``ScaledRows`` (the gate/up product finishes the norm).  ``then``:
        a norm's ``fold_request`` for the down projection (see ``Attention.forward``)."""
        if self.separate:
            x = x.materialize() if isinstance(x, ops.ScaledRows) else x
            gate_up = linear(x, self.w_gate_up, out_dtype=torch.float32)
            act = ops.gated_mul(gate_up, self.b_gate_up, self.activation, x.dtype, None, self.limit, self.alpha)
            return linear(act, self.w_down, partials_ok=True)
        act = linear(x, self.w_gate_up, epilogue=f"{self.activation}_mul")
        return linear(act, self.w_down, partials_ok=True, residual=then)


register_part("feed_forward", "swiglu", SwiGLU)
