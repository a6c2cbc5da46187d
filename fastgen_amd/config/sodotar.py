"""The Sodotar decoder as a layout of parts.

A Sodotar ``config.json`` is nested: ``width``, ``vocab``, ``norm.eps``, ``streams``, ``logit_scale`` and a list
``layers`` whose entries name their mixer (``type``: ``attention`` or ``latent_attention``), its sizes (``mixer``) and
their feed-forward (``mlp``: a mixture of experts, or null).  The model keeps ``streams`` residual streams side by
side (hyper-connections: ``l<i>.hc1.*`` for the mixer, ``l<i>.hc2.*`` for the feed-forward, each ``in [S]``, ``out [S]``
and ``mix [S, S]``); a sublayer reads a weighted sum of them through an RMS norm (``l<i>.norm1``, ``norm2``).  The
head is the embedding table, and the logits are multiplied by ``logit_scale``.

* ``attention`` is differential attention: two score maps a head over one value (``mixer.diff``: the constant of
  its ``lam``; ``lq1``, ``lk1``, ``lq2``, ``lk2``), grouped heads, rotation of the first ``rot.dims`` dimensions of each
  map (pairs ``i, i + dims/2``), and a mask of blocks: a token sees the keys before it inside its own block of
  ``mask.size`` positions.  ``kv_from: j`` makes a layer read layer ``j``'s keys and values.
* ``latent_attention`` caches one normed latent and one rotated key part a token; the heads' queries come from one
  projection (``q``); the softmax has a sink per head.
* ``mlp``: ``router.experts`` experts of width ``expert.ff`` of which a token uses ``router.top``, scores the softmax over
  all experts, choice by score + ``correction``; the experts' activation is limited by ``expert.limit``; a shared
  expert (``shared.ff``, ``shared.limit``) with a sigmoid gate of its own (``shared.sg``).

Tensors are named ``embed``, ``l<i>.mix.*``, ``l<i>.mlp.{router,correction,e<j>.{gate,up,down},shared.*}``,
``final.norm``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Mapping, Optional, Tuple, Union

from .buderax import _get
from .layout import LayerSpec, ModelLayout, PartSpec, RunEntry
from .model_args import ConfigError
from .registry import register_architecture

SWISH_ALPHA = 1.702  # the experts' activation is g * sigmoid(1.702 g) * (u + 1)


@dataclass(frozen=True)
class DiffAttentionArgs:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    block: Optional[int]
    rot_dims: int
    rot_base: float
    kv_from: Optional[int]


@dataclass(frozen=True)
class LatentArgs:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float


@dataclass(frozen=True)
class ExpertsArgs:
    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: Optional[int]
    shared_limit: Optional[float]


@dataclass(frozen=True)
class SodotarLayer:
    type: str
    mixer: Union[DiffAttentionArgs, LatentArgs]
    mlp: Optional[ExpertsArgs]


@dataclass(frozen=True)
class SodotarArgs:
    architecture: str
    width: int
    vocab: int
    norm_eps: float
    streams: int
    hyper: bool  # whether the layers have hyper-connection tensors (a model of one stream may have none)
    logit_scale: float
    layers: Tuple[SodotarLayer, ...]
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @property
    def vocab_size(self) -> int:
        return self.vocab


def _positive(where: str, **values) -> None:
    for name, v in values.items():
        if not v > 0:
            raise ConfigError(f"config.json: {where}.{name}={v} must be positive")


class SodotarArchitecture:
    name = "Sodotar"

    def parse(self, config: Mapping[str, Any], shape_of: Optional[Callable[[str], Optional[Tuple[int, ...]]]] = None
              ) -> SodotarArgs:
        layers = []
        for i, l in enumerate(_get(config, "layers")):
            kind, m, where = _get(l, "type", str), _get(l, "mixer"), f"layers[{i}].mixer"
            if kind == "attention":
                a = DiffAttentionArgs(
                    _get(m, "heads", int), _get(m, "kv_heads", int), _get(m, "dim", int), _get(m, "vdim", int),
                    _get(m, "scale", float), _get(m, "diff", float), _get(m, "mask.size", int, None),
                    _get(m, "rot.dims", int, 0), _get(m, "rot.base", float, 10000.0), _get(m, "kv_from", int, None))
                _positive(where, heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim)
                if a.heads % a.kv_heads:
                    raise ConfigError(f"config.json: {where}: heads={a.heads} is not a multiple of kv_heads={a.kv_heads}")
                if a.block is not None and a.block <= 0:
                    raise ConfigError(f"config.json: {where}.mask.size={a.block} must be positive")
                if a.rot_dims % 2 or not 0 <= a.rot_dims <= a.dim:
                    raise ConfigError(f"config.json: {where}: rot.dims={a.rot_dims} must be even and at most dim={a.dim}")
                if a.kv_from is not None:
                    j = a.kv_from
                    if not 0 <= j < i or layers[j].type != "attention" or layers[j].mixer.kv_from is not None:
                        raise ConfigError(f"config.json: {where}.kv_from={j} must name an earlier attention layer"
                                          " with keys and values of its own")
                    o = layers[j].mixer
                    if (o.kv_heads, o.dim, o.vdim, o.rot_dims, o.rot_base) != (a.kv_heads, a.dim, a.vdim, a.rot_dims, a.rot_base):
                        raise ConfigError(f"config.json: {where}: kv_heads, dim, vdim and rot must equal layer {j}'s")
            elif kind == "latent_attention":
                a = LatentArgs(_get(m, "heads", int), _get(m, "dim", int), _get(m, "rot_dim", int), _get(m, "vdim", int),
                               _get(m, "kv_rank", int), _get(m, "scale", float), _get(m, "rot.base", float))
                _positive(where, heads=a.heads, dim=a.dim, rot_dim=a.rot_dim, vdim=a.vdim, kv_rank=a.kv_rank)
                dims = _get(m, "rot.dims", int, a.rot_dim)
                if dims != a.rot_dim or a.rot_dim % 2:
                    raise ConfigError(f"config.json: {where}: rot.dims={dims} must equal rot_dim={a.rot_dim}, an even number")
            else:
                raise ConfigError(f"config.json: layers[{i}].type {kind!r} is not supported"
                                  " (supported: 'attention', 'latent_attention')")
            mlp, ff = l.get("mlp"), None
            if mlp is not None:
                where = f"layers[{i}].mlp"
                if mlp.get("kind", "moe") != "moe":
                    raise ConfigError(f"config.json: {where}.kind {mlp.get('kind')!r} is not supported (supported: 'moe')")
                ff = ExpertsArgs(_get(mlp, "router.experts", int), _get(mlp, "router.top", int), _get(mlp, "expert.ff", int),
                                 _get(mlp, "expert.limit", float), _get(mlp, "shared.ff", int, None),
                                 _get(mlp, "shared.limit", float, None))
                _positive(where, experts=ff.experts, top=ff.top, ff=ff.ff, limit=ff.limit)
                if ff.top > ff.experts:
                    raise ConfigError(f"config.json: {where}: router.top={ff.top} is more than the {ff.experts} experts")
                if ff.shared_ff is not None:
                    if ff.shared_limit is None:
                        raise ConfigError(f"config.json: required key '{where}.shared.limit' is missing")
                    _positive(where, shared_ff=ff.shared_ff, shared_limit=ff.shared_limit)
            layers.append(SodotarLayer(kind, a, ff))
        streams = _get(config, "streams", int, 1)
        if streams < 1:
            raise ConfigError(f"config.json: streams={streams} must be positive")
        hyper = streams > 1 or (shape_of is not None and shape_of("l0.hc1.in") is not None) or bool(config.get("hyper", False))
        return SodotarArgs(
            architecture=self.name, width=_get(config, "width", int), vocab=_get(config, "vocab", int),
            norm_eps=_get(config, "norm.eps", float), streams=streams, hyper=hyper,
            logit_scale=_get(config, "logit_scale", float, 1.0), layers=tuple(layers),
            extra={k: config[k] for k in ("bos_token_id", "eos_token_id") if k in config},
        )

    def to_hf_config(self, args: SodotarArgs) -> dict:
        def mixer(l: SodotarLayer) -> dict:
            m = l.mixer
            if l.type == "attention":
                out = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                       "diff": m.diff, "rot": {"base": m.rot_base, "dims": m.rot_dims}}
                if m.block is not None:
                    out["mask"] = {"size": m.block}
                if m.kv_from is not None:
                    out["kv_from"] = m.kv_from
                return out
            return {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                    "scale": m.scale, "rot": {"base": m.rot_base, "dims": m.rot_dim}}

        def mlp(f: Optional[ExpertsArgs]) -> Optional[dict]:
            if f is None:
                return None
            out = {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit}, "router": {"experts": f.experts, "top": f.top}}
            if f.shared_ff is not None:
                out["shared"] = {"ff": f.shared_ff, "limit": f.shared_limit}
            return out

        out = {"architecture": self.name, "width": args.width, "vocab": args.vocab, "norm": {"eps": args.norm_eps},
               "streams": args.streams, "logit_scale": args.logit_scale,
               "layers": [{"type": l.type, "mixer": mixer(l), "mlp": mlp(l.mlp)} for l in args.layers]}
        if args.hyper and args.streams == 1:
            out["hyper"] = True
        out.update(args.extra)
        return out

    def layout(self, args: SodotarArgs) -> ModelLayout:
        bare = {"weight": ""}  # a part's one tensor is named by the prefix alone
        D, eps = args.width, args.norm_eps

        def norm(prefix: str) -> PartSpec:
            return PartSpec("rmsnorm", prefix, dict(dim=D, eps=eps, names=bare))

        gated = {"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"}
        layers, order = [], []
        for i, l in enumerate(args.layers):
            m, p = l.mixer, f"l{i}.mix"
            reads = None
            if l.type == "attention":
                own = m.kv_from is None
                reads = None if own else m.kv_from
                rope = (PartSpec("rope", options=dict(head_dim=m.dim, rotary_dim=m.rot_dims, theta=m.rot_base, pairing="half"))
                        if m.rot_dims else PartSpec("none"))
                mixer = PartSpec("differential_attention", p, dict(
                    dim=D, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, v_head_dim=m.vdim, scale=m.scale,
                    lambda_init=m.diff, eps=eps, block=m.block, position=rope, has_kv=own, exact_weights=True,
                    names={"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "o_proj.weight": "o",
                           "lambda_q1": "lq1", "lambda_k1": "lk1", "lambda_q2": "lq2", "lambda_k2": "lk2"}))
            else:
                rope = PartSpec("rope", options=dict(head_dim=m.rot_dim, rotary_dim=m.rot_dim, theta=m.rot_base,
                                                     pairing="half"))
                mixer = PartSpec("latent_attention", p, dict(
                    dim=D, n_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, v_head_dim=m.vdim, kv_rank=m.kv_rank,
                    q_rank=None, scale=m.scale, sink=True, head_gate=False, eps=eps, position=rope, exact_weights=True,
                    names={"q_proj.weight": "q", "kv_down.weight": "dkv", "kv_down_norm.weight": "dkv.norm",
                           "k_up.weight": "uk", "v_up.weight": "uv", "sinks": "sink", "o_proj.weight": "o"}))
            f, ffn = l.mlp, None
            if f is not None:
                ffn = PartSpec("moe", f"l{i}.mlp", dict(
                    dim=D, hidden_dim=f.ff, n_experts=f.experts, top=f.top, router_bias=False, scoring="softmax_all",
                    correction=True, activation="limited", limit=f.limit, alpha=SWISH_ALPHA,
                    shared_hidden_dim=f.shared_ff, shared_activation="limited", shared_limit=f.shared_limit,
                    shared_gate=f.shared_ff is not None,
                    names={"router.weight": "router", "expert": "e{}", "shared_gate.weight": "shared.sg", **gated}))
            # (one stream without tensors of its own is the plain pre-norm layer: x <- x + sublayer(norm(x)))
            hyper = PartSpec("hyper_connections", f"l{i}", dict(streams=args.streams, dim=D, learned=args.hyper))
            layers.append(LayerSpec(mixer=mixer, ffn=ffn, mixer_norm=norm(f"l{i}.norm1"),
                                    ffn_norm=norm(f"l{i}.norm2") if ffn is not None else None,
                                    arrangement="hyper_connections", arrangement_spec=hyper))
            order.append(RunEntry(i, reads_cache_of=reads))
        return ModelLayout(
            dim=D, vocab_size=args.vocab,
            embed=PartSpec("embedding", "embed", dict(vocab_size=args.vocab, dim=D, names=bare)),
            layers=tuple(layers), order=tuple(order), final_norm=norm("final.norm"),
            head=PartSpec("lm_head", "head", dict(vocab_size=args.vocab, dim=D, tied_to="embed", names=bare,
                                                  scale=args.logit_scale)),
            streams=args.streams,
        )


SODOTAR = register_architecture(SodotarArchitecture())
