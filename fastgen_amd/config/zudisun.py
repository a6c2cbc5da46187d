"""The Zudisun decoder as a layout of parts.

A Zudisun ``config.json`` is nested: ``width``, ``vocab``, ``norm.eps`` and a list ``layers`` whose entries name
their mixer (``type``: ``attention`` or ``mamba1``), its sizes (``mixer``) and their feed-forward (``mlp``:
``{"kind": "dense", "ff": n}``, ``{"kind": "moe", "expert": {"ff": n}, "router": {...}, "shared": {"ff": n}}`` or
null).  A layer norms its sublayers' outputs only: the sublayers read the residual stream itself
(``l<i>.norm1`` behind the mixer, ``l<i>.norm2`` behind the feed-forward).  Tensors are named ``embed``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.

* ``attention``: grouped heads (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``) without rotation, with sigmoid
  weights, unit-normed queries and keys, a query temperature (``q_temp.coef``, ``q_temp.every``), a bucketed
  distance bias (``bias_max``: the distance at which the table ``mix.rel`` reaches its last row; the number of its
  rows is the tensor's shape, or the optional key ``bias_rows`` where there are no tensors yet), mixed heads
  (``mix.talk``), a bias (``mix.pb``) and an output gate (``mix.g``) per head, and, with ``v_mix``, values blended
  with those of the first such layer (``mix.vmix``).
* ``mamba1``: a selective scan (``inner``, ``state``, ``dt_rank``, ``conv`` taps).
* the dense feed-forward is gated with ReLU and has biases (``.b``); the routed one scores its experts by
  sigmoids (``router.experts``, ``top``, ``scale``, ``groups.count``, ``groups.keep``; ``mlp.correction``) and may
  have a shared expert.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Mapping, Optional, Tuple, Union

from .buderax import _get
from .layout import LayerSpec, ModelLayout, PartSpec, RunEntry
from .model_args import ConfigError
from .registry import register_architecture

DEFAULT_BIAS_ROWS = 32


@dataclass(frozen=True)
class SigmoidAttentionArgs:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp_coef: float
    q_temp_every: int
    bias_max: float
    bias_rows: int
    v_mix: bool
    vmix_stored: bool = False  # the checkpoint holds ``mix.vmix`` although the layer does not mix its values


@dataclass(frozen=True)
class MambaArgs:
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclass(frozen=True)
class DenseArgs:
    ff: int


@dataclass(frozen=True)
class RoutedArgs:
    experts: int
    top: int
    ff: int
    groups: int
    keep: int
    scale: float
    shared_ff: Optional[int]


@dataclass(frozen=True)
class ZudisunLayer:
    type: str
    mixer: Union[SigmoidAttentionArgs, MambaArgs]
    mlp: Union[None, DenseArgs, RoutedArgs]


@dataclass(frozen=True)
class ZudisunArgs:
    architecture: str
    width: int
    vocab: int
    norm_eps: float
    layers: Tuple[ZudisunLayer, ...]
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @property
    def vocab_size(self) -> int:
        return self.vocab


def _positive(where: str, **values) -> None:
    for name, v in values.items():
        if not v > 0:
            raise ConfigError(f"config.json: {where}.{name}={v} must be positive")


class ZudisunArchitecture:
    name = "Zudisun"

    def parse(self, config: Mapping[str, Any], shape_of: Optional[Callable[[str], Optional[Tuple[int, ...]]]] = None
              ) -> ZudisunArgs:
        """``shape_of(name)``: the shape of a tensor of the checkpoint (None if it has none of that name);
        sizes that only the tensors give are read from it."""
        layers = []
        first_mix: Optional[SigmoidAttentionArgs] = None
        for i, l in enumerate(_get(config, "layers")):
            kind, m, where = _get(l, "type", str), _get(l, "mixer"), f"layers[{i}].mixer"
            if kind == "attention":
                rows = _get(m, "bias_rows", int, DEFAULT_BIAS_ROWS)
                shape = shape_of(f"l{i}.mix.rel") if shape_of is not None else None
                if shape is not None:
                    rows = int(shape[0])
                a = SigmoidAttentionArgs(
                    _get(m, "heads", int), _get(m, "kv_heads", int), _get(m, "dim", int), _get(m, "vdim", int),
                    _get(m, "scale", float), _get(m, "q_temp.coef", float, 0.0), _get(m, "q_temp.every", int, 0),
                    _get(m, "bias_max", float), rows, bool(m.get("v_mix", False)),
                    shape_of is not None and shape_of(f"l{i}.mix.vmix") is not None)
                _positive(where, heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim)
                if a.heads % a.kv_heads:
                    raise ConfigError(f"config.json: {where}: heads={a.heads} is not a multiple of kv_heads={a.kv_heads}")
                if a.q_temp_every < 0 or (a.q_temp_coef != 0.0 and a.q_temp_every == 0):
                    raise ConfigError(f"config.json: {where}.q_temp.every must be positive")
                if a.bias_rows < 2 or not a.bias_max > a.bias_rows // 2:
                    raise ConfigError(f"config.json: {where}: bias_max={a.bias_max} must lie beyond half of the"
                                      f" distance table's {a.bias_rows} rows")
                if a.v_mix:
                    if first_mix is None:
                        first_mix = a
                    elif (first_mix.kv_heads, first_mix.vdim) != (a.kv_heads, a.vdim):
                        raise ConfigError(f"config.json: {where}: layers that mix values must agree in kv_heads and vdim")
            elif kind == "mamba1":
                a = MambaArgs(_get(m, "inner", int), _get(m, "state", int), _get(m, "dt_rank", int), _get(m, "conv", int))
                _positive(where, inner=a.inner, state=a.state, dt_rank=a.dt_rank, conv=a.conv)
            else:
                raise ConfigError(f"config.json: layers[{i}].type {kind!r} is not supported (supported: 'attention', 'mamba1')")
            mlp, ff, where = l.get("mlp"), None, f"layers[{i}].mlp"
            if mlp is not None:
                ff_kind = mlp.get("kind", "dense")
                if ff_kind == "dense":
                    ff = DenseArgs(_get(mlp, "ff", int))
                    _positive(where, ff=ff.ff)
                elif ff_kind == "moe":
                    groups = _get(mlp, "router.groups.count", int, 1)
                    ff = RoutedArgs(_get(mlp, "router.experts", int), _get(mlp, "router.top", int), _get(mlp, "expert.ff", int),
                                    groups, _get(mlp, "router.groups.keep", int, groups), _get(mlp, "router.scale", float, 1.0),
                                    _get(mlp, "shared.ff", int, None))
                    _positive(where, experts=ff.experts, top=ff.top, ff=ff.ff, groups=ff.groups, keep=ff.keep)
                    if ff.shared_ff is not None:
                        _positive(where, shared_ff=ff.shared_ff)
                    if ff.experts % ff.groups or ff.keep > ff.groups or ff.top > ff.keep * (ff.experts // ff.groups):
                        raise ConfigError(f"config.json: {where}: {ff.groups} groups of which {ff.keep} stay do not fit"
                                          f" {ff.experts} experts and top={ff.top}")
                else:
                    raise ConfigError(f"config.json: {where}.kind {ff_kind!r} is not supported (supported: 'dense', 'moe')")
            layers.append(ZudisunLayer(kind, a, ff))
        return ZudisunArgs(
            architecture=self.name, width=_get(config, "width", int), vocab=_get(config, "vocab", int),
            norm_eps=_get(config, "norm.eps", float), layers=tuple(layers),
            extra={k: config[k] for k in ("bos_token_id", "eos_token_id") if k in config},
        )

    def to_hf_config(self, args: ZudisunArgs) -> dict:
        def mixer(l: ZudisunLayer) -> dict:
            m = l.mixer
            if l.type == "attention":
                return {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                        "q_temp": {"coef": m.q_temp_coef, "every": m.q_temp_every}, "bias_max": m.bias_max,
                        "bias_rows": m.bias_rows, "v_mix": m.v_mix}
            return {"inner": m.inner, "state": m.state, "dt_rank": m.dt_rank, "conv": m.conv}

        def mlp(f) -> Optional[dict]:
            if f is None:
                return None
            if isinstance(f, DenseArgs):
                return {"kind": "dense", "ff": f.ff}
            return {"kind": "moe", "expert": {"ff": f.ff},
                    "router": {"experts": f.experts, "top": f.top, "scale": f.scale,
                               "groups": {"count": f.groups, "keep": f.keep}},
                    "shared": None if f.shared_ff is None else {"ff": f.shared_ff}}

        out = {"architecture": self.name, "width": args.width, "vocab": args.vocab, "norm": {"eps": args.norm_eps},
               "layers": [{"type": l.type, "mixer": mixer(l), "mlp": mlp(l.mlp)} for l in args.layers]}
        out.update(args.extra)
        return out

    def layout(self, args: ZudisunArgs) -> ModelLayout:
        bare = {"weight": ""}  # a part's one tensor is named by the prefix alone
        D, eps = args.width, args.norm_eps

        def norm(prefix: str) -> PartSpec:
            return PartSpec("rmsnorm", prefix, dict(dim=D, eps=eps, names=bare))

        gated = {"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"}
        layers = []
        for i, l in enumerate(args.layers):
            m, p = l.mixer, f"l{i}.mix"
            if l.type == "attention":
                mixer = PartSpec("sigmoid_attention", p, dict(
                    dim=D, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, v_head_dim=m.vdim, scale=m.scale,
                    eps=eps, q_temp_coef=m.q_temp_coef, q_temp_every=m.q_temp_every, bias_far=m.bias_max,
                    bias_rows=m.bias_rows, head_mix=True, head_bias=True, head_gate=True, value_mix=m.v_mix,
                    value_mix_stored=m.vmix_stored,
                    names={"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "o_proj.weight": "o",
                           "gate_proj.weight": "g", "distance_bias": "rel", "value_mix": "vmix", "head_mix": "talk",
                           "head_bias": "pb"}))
            else:
                mixer = PartSpec("selective_scan", p, dict(
                    dim=D, inner=m.inner, state=m.state, dt_rank=m.dt_rank, taps=m.conv,
                    names={"in_proj.weight": "in", "conv.weight": "conv", "conv.bias": "conv.b", "x_proj.weight": "x",
                           "dt_proj.weight": "dt", "dt_proj.bias": "dt.b", "out_proj.weight": "o"}))
            f, ffn = l.mlp, None
            if isinstance(f, DenseArgs):
                ffn = PartSpec("swiglu", f"l{i}.mlp", dict(
                    dim=D, hidden_dim=f.ff, activation="relu", bias=True,
                    names={**gated, "gate_proj.bias": "gate.b", "up_proj.bias": "up.b", "down_proj.bias": "down.b"}))
            elif isinstance(f, RoutedArgs):
                ffn = PartSpec("moe", f"l{i}.mlp", dict(
                    dim=D, hidden_dim=f.ff, n_experts=f.experts, top=f.top, router_bias=False, scoring="sigmoid",
                    correction=True, n_groups=f.groups, keep_groups=f.keep, weight_scale=f.scale,
                    shared_hidden_dim=f.shared_ff, names={"router.weight": "router", "expert": "e{}", **gated}))
            layers.append(LayerSpec(mixer=mixer, ffn=ffn, mixer_norm=norm(f"l{i}.norm1"),
                                    ffn_norm=norm(f"l{i}.norm2") if ffn is not None else None, arrangement="norm_behind"))
        return ModelLayout(
            dim=D, vocab_size=args.vocab,
            embed=PartSpec("embedding", "embed", dict(vocab_size=args.vocab, dim=D, names=bare)),
            layers=tuple(layers), order=tuple(RunEntry(i) for i in range(len(layers))), final_norm=norm("final.norm"),
            head=PartSpec("lm_head", "head", dict(vocab_size=args.vocab, dim=D, tied_to=None, names=bare)),
        )


ZUDISUN = register_architecture(ZudisunArchitecture())
