"""A selective state-space mixer (the recurrence of Mamba): a state per channel instead of a cache of keys.

``W_in x = [u | z]`` (``inner`` channels each).  ``u`` goes through a short causal convolution per channel
(``taps`` taps and a bias; the last tap meets the token itself) and SiLU.  ``W_x u = [r | B | C]`` (``dt_rank``,
``state`` and ``state`` wide); the step size of channel ``c`` is ``d_c = softplus(W_dt r + b)_c``.  With
``A = -exp(A_log)`` (``[inner, state]``) the state moves as ``S[c, n] <- exp(d_c A[c, n]) S[c, n] + d_c u_c B_n`` and
gives ``y_c = sum_n S[c, n] C_n + D_c u_c``; the output is ``W_o (y * silu(z))``.

The request's state slot holds, per channel, one fp32 row: the ``state`` values of ``S`` and behind them the last
``taps - 1`` inputs of the convolution, so that a prompt may be cut anywhere.  Step sizes, decays, the state and
the sums over it are fp32 (``csrc/selective_scan.hip``); the projections and the convolution's output have the
activation dtype.  What a token gets depends on its sequence's earlier tokens alone.

Options: ``dim``, ``inner``, ``state``, ``dt_rank``, ``taps``.
"""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, VECTOR, LayerStore, Mixer, StateNeed, TensorSpec, place, register_part

MAX_TAPS = 16
MAX_STATE = 1024


class SelectiveScan(Mixer):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.inner = int(o["inner"])
        self.state = int(o["state"])
        self.dt_rank = int(o["dt_rank"])
        self.taps = int(o["taps"])
        if min(self.inner, self.state, self.dt_rank) <= 0 or not 1 <= self.taps <= MAX_TAPS or self.state > MAX_STATE:
            raise ValueError(f"{self.prefix}: sizes must be positive, at most {MAX_TAPS} taps and {MAX_STATE} states a channel")
        # the narrow projection's rows [r | B | C], with zero rows up to a multiple of 8 (what the products' kernels read at once)
        self.narrow = -(-(self.dt_rank + 2 * self.state) // 8) * 8
        self.w_in: Optional[StreamedMatrix] = None
        self.w_x: Optional[StreamedMatrix] = None
        self.w_dt: Optional[StreamedMatrix] = None
        self.wo: Optional[StreamedMatrix] = None
        self.conv_w = self.conv_b = self.dt_bias = self.A = self.D = None

    def tensor_specs(self) -> List[TensorSpec]:
        C, N, R = self.inner, self.state, self.dt_rank
        return [
            TensorSpec(self._name("in_proj.weight"), (2 * C, self.dim)),
            TensorSpec(self._name("conv.weight"), (C, self.taps), VECTOR, ("normal", 0.3)),
            TensorSpec(self._name("conv.bias"), (C,), VECTOR, ("normal", 0.1)),
            TensorSpec(self._name("x_proj.weight"), (R + 2 * N, C), MATRIX, ("normal", 0.05)),
            TensorSpec(self._name("dt_proj.weight"), (C, R), MATRIX, ("normal", 0.1)),
            TensorSpec(self._name("dt_proj.bias"), (C,), VECTOR, ("normal", 0.5)),
            TensorSpec(self._name("A_log"), (C, N), VECTOR, ("normal", 0.5)),
            TensorSpec(self._name("D"), (C,), VECTOR, ("one_plus_normal", 0.1)),
            TensorSpec(self._name("out_proj.weight"), (self.dim, C)),
        ]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        C, N, R = self.inner, self.state, self.dt_rank
        t = lambda name: tensors[self._name(name)]
        f32 = lambda name: t(name).to(device=device, dtype=torch.float32).contiguous()
        self.w_in = streamed(place(t("in_proj.weight"), MATRIX, dtype, device))
        wx, wdt = t("x_proj.weight"), t("dt_proj.weight")
        pad = self.narrow - (R + 2 * N)
        # zero rows behind [r | B | C], and zero columns of the step projection for all but r: it reads the whole narrow row
        wx = torch.cat([wx, wx.new_zeros(pad, C)])
        wdt = torch.cat([wdt, wdt.new_zeros(C, self.narrow - R)], dim=1)
        self.w_x = streamed(place(wx, MATRIX, dtype, device))
        self.w_dt = streamed(place(wdt, MATRIX, dtype, device))
        self.wo = streamed(place(t("out_proj.weight"), MATRIX, dtype, device))
        self.conv_w, self.conv_b, self.dt_bias, self.D = f32("conv.weight"), f32("conv.bias"), f32("dt_proj.bias"), f32("D")
        self.A = (-torch.exp(f32("A_log"))).contiguous()

    def state_need(self) -> StateNeed:
        return StateNeed((self.inner, self.state + self.taps - 1), torch.float32)

    def forward(self, x: torch.Tensor, ctx: Any, store: LayerStore) -> torch.Tensor:
        C, N, R = self.inner, self.state, self.dt_rank
        T = x.shape[0]
        rows = linear(x, self.w_in)  # [T, u | z]
        u = torch.empty((T, C), dtype=x.dtype, device=x.device)
        ops.causal_conv(rows, self.conv_w, self.conv_b, store.state, N, ctx.slot_ids, ctx.seq_of_token, ctx.q_start, u,
                        activation="silu")
        narrow = linear(u, self.w_x)  # [T, r | B | C | zeros]
        dt = linear(narrow, self.w_dt, out_dtype=torch.float32)
        y = torch.empty((T, C), dtype=x.dtype, device=x.device)
        ops.selective_scan(u, dt, self.dt_bias, self.A, narrow, R, R + N, self.D, rows[:, C:], rows, self.taps,
                           store.state, ctx.slot_ids, ctx.q_start, ctx.n_seqs, y,
                           q_start_host=None if ctx.graph_capacity else ctx.q_start_host)
        return linear(y, self.wo, partials_ok=True)


register_part("mixer", "selective_scan", SelectiveScan)
