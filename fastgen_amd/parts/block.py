"""Arrangements: how a layer's mixer, feed-forward and norms are wired to
the residual stream."""

from __future__ import annotations

from typing import Any, Optional

import torch

from ..kernels import ops
from ..kernels.ops import ScaledRows
from .base import VECTOR, FeedForward, LayerStore, Mixer, Norm, Part, TensorSpec, register_part


def _no_output_bias(ffn, arrangement: str) -> None:
    """Only an arrangement that norms a feed-forward's output adds a bias of its last projection."""
    if ffn is not None and getattr(ffn, "bias", False):
        raise ValueError(f"a {arrangement} layer does not take a feed-forward with biases")


class PreNormBlock:
    """``h += mixer(norm(h)); h += ffn(norm(h))`` (``fastgen/forward.py:419-499``).

    The residual stream ``h`` is fp32.  Each addition is done by the norm
    that follows it, so a block takes the previous block's output as
    ``pending`` and returns its feed-forward's output un-added.

    For few rows the norms need no kernels of their own: a part that says so (``folds_norms``) is
    handed the norm that follows it (``then``) and may add its output to ``h`` and half-do that norm
    in its last product; it then returns ``ScaledRows`` instead of rows to be added, and the part
    after it finishes the norm in its first product.  ``next_norm`` is the norm that follows this
    block (the next block's first); a ``pending`` that is ``ScaledRows`` was made for this block's
    first norm.  Every step of this is optional: what a part does not fold, the norm's kernel does.
    """

    folds_norms = True

    def __init__(self, mixer: Mixer, ffn: FeedForward, mixer_norm: Norm, ffn_norm: Norm) -> None:
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm
        _no_output_bias(ffn, "pre-norm")

    @staticmethod
    def _run(part, x, then, *args):
        """``part.forward`` with what it understands: ScaledRows and ``then`` only if it folds norms."""
        if getattr(part, "folds_norms", False):
            return part.forward(x, *args, then=then)
        return part.forward(x.materialize() if isinstance(x, ScaledRows) else x, *args)

    def forward(self, h: torch.Tensor, pending, ctx: Any, store: LayerStore, next_norm: Optional[Norm] = None):
        x = pending if isinstance(pending, ScaledRows) else self.mixer_norm.forward(h, pending, ctx.act_dtype)
        then = self.ffn_norm.fold_request(h) if hasattr(self.ffn_norm, "fold_request") else None
        mixed = self._run(self.mixer, x, then, ctx, store)
        x = mixed if isinstance(mixed, ScaledRows) else self.ffn_norm.forward(h, mixed, ctx.act_dtype)
        then = next_norm.fold_request(h) if next_norm is not None and hasattr(next_norm, "fold_request") else None
        return self._run(self.ffn, x, then)


register_part("arrangement", "pre_norm", lambda spec, *parts: PreNormBlock(*parts))


class ParallelBlock:
    """``x = norm(h); h += mixer(x) + ffn(x)``: one norm, both sublayers read its output, and their
    sum (taken first, in fp32) goes to the residual stream.  A layer without a feed-forward adds its
    mixer's output alone.  Like the other arrangements it leaves the addition to whatever norm
    follows: it takes the layer before's output as ``pending`` and returns its own un-added.

    A feed-forward that can take the mixer's output into its last kernel (``adds_to``) returns the
    sum as fp32 ``[1, T, dim]``; any other feed-forward's rows are added by a kernel of their own.
    """

    folds_norms = False

    def __init__(self, mixer: Mixer, ffn: Optional[FeedForward], mixer_norm: Norm, ffn_norm: Optional[Norm] = None) -> None:
        if ffn_norm is not None:
            raise ValueError("a parallel layer has one norm: its feed-forward reads the mixer's")
        self.mixer, self.ffn, self.mixer_norm = mixer, ffn, mixer_norm
        _no_output_bias(ffn, "parallel")

    def forward(self, h: torch.Tensor, pending, ctx: Any, store: LayerStore):
        x = self.mixer_norm.forward(h, pending, ctx.act_dtype)
        mixed = self.mixer.forward(x, ctx, store)
        if self.ffn is None:
            return mixed
        if getattr(self.ffn, "adds_to", False):
            return self.ffn.forward(x, plus=mixed)
        fed = self.ffn.forward(x)
        if mixed.dim() == 3 or fed.dim() == 3:
            # fp32 partial sums (products whose k range was cut): all of them are the norm's to add
            as_parts = lambda t: t if t.dim() == 3 else t.float()[None]
            return torch.cat([as_parts(mixed), as_parts(fed)])
        return ops.add_rows(mixed, fed)


register_part("arrangement", "parallel", lambda spec, *parts: ParallelBlock(*parts))


class SandwichBlock:
    """``h += post_mixer(mixer(norm(h))); h += post_ffn(ffn(norm(h)))``: a norm before and a norm behind every
    sublayer.  The norms behind are ``extra_norms`` of the layer, ``post_mixer`` and ``post_ffn``.  A
    sublayer's output goes on as :class:`~fastgen_amd.kernels.ops.PostNormed`: the norm that follows (this
    block's second, the next block's first, the model's last) norms it, adds it to the stream and norms
    the stream in one kernel, in fp32.  A layer without a feed-forward has only the first half."""

    folds_norms = False

    def __init__(self, mixer: Mixer, ffn: Optional[FeedForward], mixer_norm: Norm, ffn_norm: Optional[Norm],
                 extra: Optional[dict] = None) -> None:
        extra = extra or {}
        if "post_mixer" not in extra or (ffn is not None and ("post_ffn" not in extra or ffn_norm is None)):
            raise ValueError("a sandwich layer needs the norms post_mixer and, with a feed-forward, ffn_norm and post_ffn")
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm
        self.post_mixer, self.post_ffn = extra["post_mixer"], extra.get("post_ffn")
        _no_output_bias(ffn, "sandwich")

    @staticmethod
    def _behind(rows, norm) -> ops.PostNormed:
        return ops.PostNormed(rows, norm.weight, norm.eps)

    def forward(self, h: torch.Tensor, pending, ctx: Any, store: LayerStore):
        x = self.mixer_norm.forward(h, pending, ctx.act_dtype)
        mixed = self._behind(self.mixer.forward(x, ctx, store), self.post_mixer)
        if self.ffn is None:
            return mixed
        x = self.ffn_norm.forward(h, mixed, ctx.act_dtype)
        return self._behind(self.ffn.forward(x), self.post_ffn)


register_part("arrangement", "sandwich", lambda spec, *parts: SandwichBlock(*parts))


class NormBehindBlock:
    """``h += norm1(mixer(h)); h += norm2(ffn(h))``: the sublayers read the residual stream itself (rounded to the
    activation dtype) and only their outputs are normed.  ``mixer_norm`` and ``ffn_norm`` are the norms behind the
    mixer and the feed-forward.  One kernel norms what the sublayer before gave, adds it to the fp32 stream and
    stores the stream's rows for the next sublayer.  A feed-forward whose last projection has a bias
    (``output_bias``) leaves it to that kernel, which adds it in fp32 before the norm.  A layer without a
    feed-forward has only the first half."""

    folds_norms = False

    def __init__(self, mixer: Mixer, ffn: Optional[FeedForward], mixer_norm: Norm, ffn_norm: Optional[Norm]) -> None:
        if ffn is not None and ffn_norm is None:
            raise ValueError("a feed-forward whose output is normed needs its norm")
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm

    @staticmethod
    def _stream_rows(h: torch.Tensor, pending, dtype: torch.dtype) -> torch.Tensor:
        """Add ``pending`` to the stream and return the stream's rows in ``dtype``."""
        x = torch.empty(h.shape, dtype=dtype, device=h.device)
        if isinstance(pending, ops.PostNormed):
            return ops.post_add_rmsnorm(h, pending.rows, pending.weight, pending.eps, None, 0.0, x, delta_bias=pending.bias)
        if pending is not None:
            ops.stream_add(h, pending, None, None)
        return ops.post_add_rmsnorm(h, None, None, 0.0, None, 0.0, x)

    def forward(self, h: torch.Tensor, pending, ctx: Any, store: LayerStore):
        x = self._stream_rows(h, pending, ctx.act_dtype)
        mixed = ops.PostNormed(self.mixer.forward(x, ctx, store), self.mixer_norm.weight, self.mixer_norm.eps)
        if self.ffn is None:
            return mixed
        x = self._stream_rows(h, mixed, ctx.act_dtype)
        return ops.PostNormed(self.ffn.forward(x), self.ffn_norm.weight, self.ffn_norm.eps,
                              getattr(self.ffn, "output_bias", None))


register_part("arrangement", "norm_behind", lambda spec, *parts: NormBehindBlock(*parts))


class HyperConnectionBlock(Part):
    """Several residual streams side by side.  The model keeps ``streams`` copies ``X[0..S-1]`` of the residual
    stream (fp32 ``[S, T, dim]``; all equal the embedding's output at the start, and the model's last norm reads
    their sum).  Each sublayer ``q`` (1: the mixer, 2: the feed-forward) has three small tensors, ``hc<q>.in [S]``,
    ``hc<q>.out [S]`` and ``hc<q>.mix [S, S]`` (from-stream by to-stream):

        u = sum_s in[s] X[s];  y = sublayer(norm(u));  X'[t] = sum_s mix[s, t] X[s] + out[t] y   (all t at once)

    As the other arrangements leave the addition of a sublayer's output to the norm that follows, this one
    leaves the update: a sublayer's output goes on as :class:`~fastgen_amd.kernels.ops.StreamUpdate`, and one
    kernel (``ops.streams_step``) applies it, forms the next ``u`` and norms it, all in fp32.  A layer without a
    feed-forward has the first half only.  Options: ``streams``, ``dim``, ``learned`` (False: there are no such
    tensors, every weight is one: with one stream that is the plain pre-norm layer); the spec's prefix is the
    layer's."""

    folds_norms = False

    def __init__(self, spec, mixer: Mixer, ffn: Optional[FeedForward], mixer_norm: Norm, ffn_norm: Optional[Norm]) -> None:
        super().__init__(spec)
        self.streams = int(spec.options["streams"])
        self.learned = bool(spec.options.get("learned", True))
        if not 1 <= self.streams <= ops.STREAMS_MAX:
            raise ValueError(f"{self.prefix}: {self.streams} streams are not supported (1 to {ops.STREAMS_MAX})")
        if ffn is not None and ffn_norm is None:
            raise ValueError("a feed-forward needs its norm")
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm
        _no_output_bias(ffn, "hyper-connection")
        self.weights: dict = {}

    def _sublayers(self):
        return ("hc1", "hc2") if self.ffn is not None else ("hc1",)

    def tensor_specs(self):
        S, specs = self.streams, []
        for q in self._sublayers() if self.learned else ():
            specs += [TensorSpec(self._name(f"{q}.in"), (S,), VECTOR, ("one_plus_normal", 0.1)),
                      TensorSpec(self._name(f"{q}.out"), (S,), VECTOR, ("one_plus_normal", 0.1)),
                      TensorSpec(self._name(f"{q}.mix"), (S, S), VECTOR, ("eye_plus_normal", 0.1))]
        return specs

    def load(self, tensors, dtype, device) -> None:
        for q in self._sublayers():
            for n in ("in", "out", "mix"):
                shape = (self.streams, self.streams) if n == "mix" else (self.streams,)
                self.weights[f"{q}.{n}"] = (tensors[self._name(f"{q}.{n}")].to(device=device, dtype=torch.float32).contiguous()
                                            if self.learned else torch.ones(shape, dtype=torch.float32, device=device))

    def _read(self, h: torch.Tensor, pending, q: str, norm: Norm, dtype: torch.dtype) -> torch.Tensor:
        if h.dim() != 3 or h.shape[0] != self.streams:
            raise ValueError(f"{self.prefix}: the model keeps no {self.streams} residual streams (ModelLayout.streams)")
        if pending is not None and not isinstance(pending, ops.StreamUpdate):
            raise ValueError(f"{self.prefix}: what the layer before left is no update of the streams")
        out = torch.empty(h.shape[1:], dtype=dtype, device=h.device)
        return ops.streams_step(h, pending, self.weights[f"{q}.in"], norm.weight, norm.eps, out)

    def forward(self, h: torch.Tensor, pending, ctx: Any, store: LayerStore):
        x = self._read(h, pending, "hc1", self.mixer_norm, ctx.act_dtype)
        update = ops.StreamUpdate(self.mixer.forward(x, ctx, store), self.weights["hc1.mix"], self.weights["hc1.out"])
        if self.ffn is None:
            return update
        x = self._read(h, update, "hc2", self.ffn_norm, ctx.act_dtype)
        return ops.StreamUpdate(self.ffn.forward(x), self.weights["hc2.mix"], self.weights["hc2.out"])


register_part("arrangement", "hyper_connections", HyperConnectionBlock)
