"""A routed feed-forward: a mixture of gated experts.

Every row goes to the ``top`` experts whose router logits are the largest
(``x W_r^T + b`` in fp32), weighted by the softmax over those logits alone; an
expert is ``W_down (silu(W_gate x) * (W_up x))`` without biases, and the output
is the weighted sum of the chosen experts' outputs, taken in fp32.  All of it
runs on the device (``csrc/moe.hip``): which rows went where is never looked
at on the host, so a step with this part can be recorded.

Options beyond that: ``scoring`` = ``"sigmoid"`` (an expert's score is the sigmoid
of its logit; the chosen experts' scores divided by their sum, times
``weight_scale``, are the weights), ``correction`` (a number per expert added to
the scores for the choice only), ``n_groups`` / ``keep_groups`` (the experts form
equal groups of neighbours and only those of the best groups can be chosen),
``shared_hidden_dim`` (a gated feed-forward of that width, ``shared``, runs for
every row and is added).  ``scoring`` = ``"softmax_all"``: the scores are the softmax
of the logits over all experts, and choice (with ``correction``) and weights go as
with sigmoid scores.  ``activation`` = ``"limited"`` with ``limit`` (and ``alpha``): an
expert is ``W_down (g * sigmoid(alpha g) * (u + 1))`` of ``g = min(W_gate x, limit)`` and
``u = clamp(W_up x, -limit, limit)``; ``shared_activation`` / ``shared_limit`` say the same
of the shared expert.  ``shared_gate``: the shared expert's output is multiplied by
``sigmoid(w . x)`` for one more row ``w`` (``shared_gate.weight [1, dim]``), whose logit the
router's kernel computes in fp32 beside the experts'.
"""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..config.layout import PartSpec
from .base import MATRIX, VECTOR, FeedForward, TensorSpec, build_part, place, register_part


class MoE(FeedForward):
    adds_to = True  # ``forward(x, plus=rows)`` returns plus + its own output, as fp32 [1, T, dim]

    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.hidden_dim = int(o["hidden_dim"])
        self.n_experts = int(o["n_experts"])
        self.top = int(o["top"])
        if not 1 <= self.top <= self.n_experts:
            raise ValueError(f"{self.prefix}: top={self.top} must be between 1 and n_experts={self.n_experts}")
        self.router_bias = bool(o.get("router_bias", True))
        self.scoring = o.get("scoring", "softmax")
        if self.scoring not in ("softmax", "sigmoid", "softmax_all"):
            raise ValueError(f"{self.prefix}: scoring {self.scoring!r} is not supported ('softmax', 'sigmoid', 'softmax_all')")
        self.activation = o.get("activation", "silu")
        self.limit, self.alpha = float(o.get("limit") or 0.0), float(o.get("alpha", 1.0))
        if self.activation not in ("silu", "limited") or (self.activation == "limited") != (self.limit > 0):
            raise ValueError(f"{self.prefix}: activation {self.activation!r} with limit={self.limit} is not supported"
                             " ('silu', or 'limited' with a positive limit)")
        self.has_correction = bool(o.get("correction", False))
        self.n_groups, self.keep_groups = int(o.get("n_groups", 1)), int(o.get("keep_groups", o.get("n_groups", 1)))
        self.weight_scale = float(o.get("weight_scale", 1.0))
        if self.scoring == "softmax" and (self.has_correction or self.n_groups != 1 or self.weight_scale != 1.0):
            raise ValueError(f"{self.prefix}: correction, groups and weight_scale go with sigmoid or softmax_all scoring")
        if (self.n_groups < 1 or self.n_experts % self.n_groups or not 1 <= self.keep_groups <= self.n_groups
                or self.top > self.keep_groups * (self.n_experts // self.n_groups)):
            raise ValueError(f"{self.prefix}: {self.n_groups} groups of which {self.keep_groups} stay do not fit"
                             f" {self.n_experts} experts and top={self.top}")
        self.correction: Optional[torch.Tensor] = None
        self.shared: Optional[FeedForward] = None
        self.shared_gate = bool(o.get("shared_gate", False))
        if o.get("shared_hidden_dim"):
            names = o.get("names", {})
            self.shared = build_part("feed_forward", PartSpec("swiglu", self._name("shared"), dict(
                dim=self.dim, hidden_dim=int(o["shared_hidden_dim"]), activation=o.get("shared_activation", "silu"),
                limit=o.get("shared_limit"), alpha=self.alpha,
                names={k: names[k] for k in ("gate_proj.weight", "up_proj.weight", "down_proj.weight") if k in names})))
        elif self.shared_gate:
            raise ValueError(f"{self.prefix}: a gate of the shared expert needs a shared expert")
        self.router: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.w_gate: Optional[torch.Tensor] = None  # [E, hidden (padded to 8), dim]
        self.w_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None  # [E, dim, hidden (padded to 8)]

    def _expert(self, e: int, which: str) -> str:
        names = self.spec.options.get("names", {})
        return self._name(f"{names.get('expert', 'experts.{}').format(e)}.{names.get(which, which)}")

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self._name("router.weight"), (self.n_experts, self.dim), MATRIX, ("normal", 0.3))]
        if self.router_bias:
            specs.append(TensorSpec(self._name("router.bias"), (self.n_experts,), VECTOR, ("normal", 0.3)))
        if self.has_correction:
            specs.append(TensorSpec(self._name("correction"), (self.n_experts,), VECTOR, ("normal", 0.1)))
        if self.shared is not None:
            specs += self.shared.tensor_specs()
        if self.shared_gate:
            specs.append(TensorSpec(self._name("shared_gate.weight"), (1, self.dim), MATRIX, ("normal", 0.3)))
        for e in range(self.n_experts):
            specs += [TensorSpec(self._expert(e, "gate_proj.weight"), (self.hidden_dim, self.dim)),
                      TensorSpec(self._expert(e, "up_proj.weight"), (self.hidden_dim, self.dim)),
                      TensorSpec(self._expert(e, "down_proj.weight"), (self.dim, self.hidden_dim))]
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        # the router's logits are fp32 whatever the model's dtype is
        router = tensors[self._name("router.weight")]
        if self.shared_gate:  # one more row behind the experts': the shared expert's gate
            router = torch.cat([router, tensors[self._name("shared_gate.weight")].to(router.dtype)])
        self.router = router.to(device=device, dtype=torch.float32).contiguous()
        if self.router_bias:
            self.bias = tensors[self._name("router.bias")].to(device=device, dtype=torch.float32).contiguous()
        if self.has_correction:
            self.correction = tensors[self._name("correction")].to(device=device, dtype=torch.float32).contiguous()
        if self.shared is not None:
            self.shared.load(tensors, dtype, device)
        gate = torch.stack([tensors[self._expert(e, "gate_proj.weight")] for e in range(self.n_experts)])
        up = torch.stack([tensors[self._expert(e, "up_proj.weight")] for e in range(self.n_experts)])
        down = torch.stack([tensors[self._expert(e, "down_proj.weight")] for e in range(self.n_experts)])
        pad = -self.hidden_dim % 8
        if pad:
            # the matrix-core kernels read k in chunks of 8: channels of zero weights are added, whose
            # activation silu(0) * 0 = 0 meets zero columns of the down projection
            gate = torch.cat([gate, gate.new_zeros(self.n_experts, pad, self.dim)], dim=1)
            up = torch.cat([up, up.new_zeros(self.n_experts, pad, self.dim)], dim=1)
            down = torch.cat([down, down.new_zeros(self.n_experts, self.dim, pad)], dim=2)
        self.w_gate = place(gate, MATRIX, dtype, device)
        self.w_up = place(up, MATRIX, dtype, device)
        self.w_down = place(down, MATRIX, dtype, device)

    def tile_rows(self, n_rows: int) -> int:
        """Rows of one expert a tile holds: 16 for few rows (decode: an expert's matrices are read once for
        its rows), more where the experts get so many rows each that their matrices would otherwise be
        read many times over; from about a hundred rows an expert the tiles that go through LDS (the
        matrix-core kernels only)."""
        if self.w_gate.dtype != torch.bfloat16 or self.dim % 8:
            return 16
        per_expert = n_rows * self.top / self.n_experts
        lds_ok = min(self.dim, self.w_down.shape[2]) >= 32  # the tiles through LDS load k in steps of 32
        # a tile is computed whole whatever it holds, and every expert's last tile is half empty on average:
        # the largest tiles only where an expert has several of them
        for rows, least in ((256, 768), (128, 96), (64, 48), (32, 24)):
            if per_expert >= least and (rows < 128 or lds_ok):
                return rows
        return 16

    def forward(self, x: torch.Tensor, plus: Optional[torch.Tensor] = None) -> torch.Tensor:
        """fp32 ``[1, T, dim]``: the experts' weighted sum (plus ``plus``, rows that go to the
        residual stream with it), for a norm to add."""
        tile_rows = self.tile_rows(x.shape[0])
        if self.shared is not None:
            both = self.shared.forward(x)
            if self.shared_gate and plus is not None:
                raise ValueError(f"{self.prefix}: a gated shared expert does not go with rows added from outside")
            plus = both if plus is None else torch.cat([t if t.dim() == 3 else t.float()[None] for t in (plus, both)])
        routed = ops.moe_route(x, self.router, self.bias, self.top, self.scoring == "sigmoid", self.correction,
                               self.n_groups, self.keep_groups, self.weight_scale,
                               softmax_scores=self.scoring == "softmax_all", n_extra=int(self.shared_gate))
        choice, weight = routed[0], routed[1]
        sorted_, tiles = ops.moe_sort(choice, self.n_experts, tile_rows)
        act = ops.moe_gate_up(x, self.w_gate, self.w_up, sorted_, tiles, self.top, tile_rows, self.limit, self.alpha)
        y = ops.moe_down(act, self.w_down, sorted_, tiles, tile_rows)
        return ops.moe_combine(y, weight, plus, routed[2][:, 0] if self.shared_gate else None)


register_part("feed_forward", "moe", MoE)
