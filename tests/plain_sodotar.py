"""A plain, slow Sodotar: whole sequences, no cache, no batching, one function
per mechanism, sharing no code with ``fastgen_amd``.  It is what the engine is
compared with.

The model (notation of this file).  Tokens are embedded; the embedding's output
is copied into ``S`` residual streams ``X[0..S-1]``.  A sublayer ``f`` (mixer, then
feed-forward) of a layer with the numbers ``a[S]`` (in), ``b[S]`` (out) and
``M[S, S]`` (mix, from-stream by to-stream) does

    u = sum_s a[s] X[s];   y = f(rms(u) * w);   X'[t] = sum_s M[s, t] X[s] + b[t] y

and after the last layer the streams are added up, normed, and multiplied with
the embedding table and a constant.  Two mixers exist:

* ``attention`` (differential): every head has two score maps (two queries, two
  keys of size ``d``) over one value; both are rotated on their first ``rot``
  dimensions (pairs ``i, i + rot/2``), see only the keys of their own block of
  ``size`` positions (blocks counted from position 0), and are softmaxed apart;
  ``o = A1 v - lam A2 v`` with ``lam = exp(lq1 . lk1) - exp(lq2 . lk2) + c``, then
  ``o`` is divided by its root mean square over the head and multiplied by
  ``1 - c``.  A layer may use an earlier layer's rotated keys and values.
* ``latent_attention``: the key/value side is one narrow normed latent ``c`` and
  one rotated part ``r`` shared by the heads; a head's key is ``[W_uk c | r]``, its
  value ``W_uv c``; causal; the softmax's denominator holds one more term
  ``exp(sink_h)``.

The feed-forward is a mixture of experts: scores are the softmax of the router's
logits over all experts, the ``top`` largest of score + correction are chosen,
weighted by their scores over the chosen ones' sum; an expert is
``W_down (g * sigmoid(1.702 g) * (u + 1))`` with ``g = min(W_gate h, L)`` and
``u = clamp(W_up h, -L, L)``; a shared expert of the same form runs for every
token, times ``sigmoid(w_sg . h)``.

``dtype`` is the precision of matrix products and activations; norms, the
streams, angles, scores and weights and routers stay in float32 (float64 when the
whole run is).
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch


def _hi(x: torch.Tensor) -> torch.Tensor:
    return x if x.dtype == torch.float64 else x.float()


def _mm(x: torch.Tensor, w: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``x W^T`` with operands in ``dtype``, summed in the high precision, rounded once to ``dtype``."""
    return (_hi(x.to(dtype)) @ _hi(w.to(dtype)).T).to(dtype)


# ------------------------------------------------------------------ mechanisms
def plain_rms(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    x = _hi(x)
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * _hi(w)


def plain_rotate(x: torch.Tensor, base: float, dims: int, first: int = 0) -> torch.Tensor:
    """``x [T, ..., d]``: the run of ``dims`` dimensions from ``first`` is turned, dimension ``i`` of the run paired
    with ``i + dims/2``, by the angle ``p * base^(-2i/dims)`` at position ``p`` (the row index)."""
    x = _hi(x).clone()
    T, half = x.shape[0], dims // 2
    p = torch.arange(T, dtype=x.dtype)
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    ang = p[:, None] * f[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., first : first + half].clone(), x[..., first + half : first + dims].clone()
    x[..., first : first + half] = u * cos - v * sin
    x[..., first + half : first + dims] = v * cos + u * sin
    return x


def plain_softmax_rows(scores: torch.Tensor, visible: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Weights of ``scores [H, T, T]`` over the ``visible [T, T]`` keys; with ``sink [H]`` the denominator has one
    more term ``exp(sink_h)``."""
    s = scores.masked_fill(~visible[None], -math.inf)
    m = s.amax(-1, keepdim=True)
    if sink is not None:
        m = torch.maximum(m, _hi(sink).to(s.dtype)[:, None, None])
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(_hi(sink).to(s.dtype)[:, None, None] - m)
    return e / den


def plain_block_mask(T: int, size: Optional[int]) -> torch.Tensor:
    """``[query, key]``: key ``j <= i`` in the same block of ``size`` positions as ``i`` (all ``j <= i`` without size)."""
    i = torch.arange(T)
    ok = i[None, :] <= i[:, None]
    if size:
        ok = ok & ((i[None, :] // size) == (i[:, None] // size))
    return ok


def plain_diff_keys(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, dtype: torch.dtype):
    """Rotated keys ``[T, G, 2, d]`` and values ``[T, G, e]`` of a differential attention layer."""
    T, G, d, e = x.shape[0], m["kv_heads"], m["dim"], m["vdim"]
    k = _mm(x, w[f"{p}.k"], dtype).view(T, G, 2, d)
    k = plain_rotate(k, m["rot"]["base"], m["rot"]["dims"]).to(dtype)
    return k, _mm(x, w[f"{p}.v"], dtype).view(T, G, e)


def plain_diff_attention(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                         dtype: torch.dtype, kv=None):
    """``x [T, D]`` -> ``[T, D]``; returns also the (keys, values) it used or made."""
    T, H, G, d, e = x.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    c = m["diff"]
    q = _mm(x, w[f"{p}.q"], dtype).view(T, H, 2, d)
    q = plain_rotate(q, m["rot"]["base"], m["rot"]["dims"]).to(dtype)
    if kv is None:
        kv = plain_diff_keys(x, w, p, m, dtype)
    k, v = kv
    lam = (torch.exp((_hi(w[f"{p}.lq1"]) * _hi(w[f"{p}.lk1"])).sum())
           - torch.exp((_hi(w[f"{p}.lq2"]) * _hi(w[f"{p}.lk2"])).sum()) + c)
    visible = plain_block_mask(T, (m.get("mask") or {}).get("size"))
    out = torch.zeros(T, H, e, dtype=_hi(x).dtype)
    for h in range(H):
        g = h // (H // G)
        maps = []
        for j in range(2):
            s = (_hi(q[:, h, j]) @ _hi(k[:, g, j]).T) * m["scale"]
            a = plain_softmax_rows(s[None], visible)[0]
            maps.append(a @ _hi(v[:, g]))
        o = maps[0] - lam.to(maps[0].dtype) * maps[1]
        out[:, h] = plain_rms(o, None, eps) * (1.0 - c)
    return _mm(out.reshape(T, H * e).to(dtype), w[f"{p}.o"], dtype), kv


def plain_latent_attention(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                           dtype: torch.dtype) -> torch.Tensor:
    T, H, d, r, e, R = x.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base = m["rot"]["base"]
    q = _mm(x, w[f"{p}.q"], dtype).view(T, H, d + r)
    q = plain_rotate(q, base, r, first=d).to(dtype)
    low = _mm(x, w[f"{p}.dkv"], dtype)
    c = plain_rms(low[:, :R], w[f"{p}.dkv.norm"], eps).to(dtype)
    shared = plain_rotate(low[:, R:], base, r).to(dtype)
    keys = _mm(c, w[f"{p}.uk"], dtype).view(T, H, d)
    vals = _mm(c, w[f"{p}.uv"], dtype).view(T, H, e)
    visible = plain_block_mask(T, None)
    s = torch.einsum("thd,jhd->htj", _hi(q[..., :d]), _hi(keys)) + torch.einsum("thd,jd->htj", _hi(q[..., d:]), _hi(shared))
    a = plain_softmax_rows(s * m["scale"], visible, w[f"{p}.sink"])
    out = torch.einsum("htj,jhe->the", a, _hi(vals))
    return _mm(out.reshape(T, H * e).to(dtype), w[f"{p}.o"], dtype)


def plain_expert(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, limit: float, dtype: torch.dtype) -> torch.Tensor:
    g = _hi(_mm(x, w[f"{p}.gate"], dtype)).clamp(max=limit)
    u = _hi(_mm(x, w[f"{p}.up"], dtype)).clamp(min=-limit, max=limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return _mm(y.to(dtype), w[f"{p}.down"], dtype)


def plain_route(x: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top: int, dtype: torch.dtype):
    """Chosen experts ``[T, top]`` and their weights: softmax over all experts, choice by score + correction
    (ties: the lower expert), weights the chosen scores over their sum."""
    s = torch.softmax(_hi(x.to(dtype)) @ _hi(router).T, dim=-1)
    pick = s + _hi(correction)
    chosen = torch.sort(pick, dim=-1, descending=True, stable=True).indices[:, :top]
    ws = torch.gather(s, 1, chosen)
    return chosen, ws / (ws.sum(-1, keepdim=True) + 1e-20)


def plain_moe(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, mlp: Mapping, dtype: torch.dtype) -> torch.Tensor:
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    chosen, ws = plain_route(x, w[f"{p}.router"], w[f"{p}.correction"], top, dtype)
    out = torch.zeros(x.shape[0], x.shape[1], dtype=_hi(x).dtype)
    for e in range(E):
        rows, slot = (chosen == e).nonzero(as_tuple=True)
        if rows.numel():
            y = _hi(plain_expert(x[rows], w, f"{p}.e{e}", mlp["expert"]["limit"], dtype))
            out.index_add_(0, rows, y * ws[rows, slot][:, None])
    if mlp.get("shared"):
        gate = torch.sigmoid(_hi(x.to(dtype)) @ _hi(w[f"{p}.shared.sg"]).T)  # [T, 1]
        out = out + gate * _hi(plain_expert(x, w, f"{p}.shared", mlp["shared"]["limit"], dtype))
    return out


def plain_streams_step(X: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, f) -> torch.Tensor:
    """One sublayer on the streams ``X [S, T, D]``: ``f`` maps the streams' weighted sum to the sublayer's output."""
    a, b, M = _hi(w[f"{p}.in"]).to(X.dtype), _hi(w[f"{p}.out"]).to(X.dtype), _hi(w[f"{p}.mix"]).to(X.dtype)
    y = f(torch.einsum("s,std->td", a, X)).to(X.dtype)
    return torch.einsum("sr,std->rtd", M, X) + b[:, None, None] * y[None]


# ----------------------------------------------------------------------- model
def plain_forward(weights: Mapping[str, torch.Tensor], config: Mapping, tokens: List[int],
                  dtype: torch.dtype = torch.float32, layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence.  ``layers_out``: a list that gets the sum of the streams after
    every layer."""
    w = {k: v if v.dtype == torch.float64 or not v.dtype.is_floating_point else v.to(dtype) for k, v in weights.items()}
    if dtype == torch.float64:
        w = {k: v.double() if v.dtype.is_floating_point else v for k, v in weights.items()}
    eps = config["norm"]["eps"]
    S = int(config.get("streams", 1))
    x = _hi(w["embed"][torch.tensor(tokens)])
    X = x[None].repeat(S, 1, 1)
    kept: Dict[int, tuple] = {}
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}"

        def mixer(u, i=i, m=m, p=p, kind=layer["type"]):
            h = plain_rms(u, w[f"{p}.norm1"], eps).to(dtype)
            if kind == "attention":
                y, kv = plain_diff_attention(h, w, f"{p}.mix", m, eps, dtype, kept.get(m.get("kv_from")))
                if m.get("kv_from") is None:
                    kept[i] = kv
                return _hi(y)
            if kind == "latent_attention":
                return _hi(plain_latent_attention(h, w, f"{p}.mix", m, eps, dtype))
            raise ValueError(kind)

        X = plain_streams_step(X, w, f"{p}.hc1", mixer)
        if layer.get("mlp") is not None:
            X = plain_streams_step(X, w, f"{p}.hc2",
                                   lambda u: plain_moe(plain_rms(u, w[f"{p}.norm2"], eps).to(dtype), w, f"{p}.mlp",
                                                       layer["mlp"], dtype))
        if layers_out is not None:
            layers_out.append(X.sum(0))
    x = plain_rms(X.sum(0), w["final.norm"], eps).to(dtype)
    return (_hi(x) @ _hi(w["embed"]).T) * config.get("logit_scale", 1.0)


def plain_greedy(weights: Mapping[str, torch.Tensor], config: Mapping, prompt: List[int], n_new: int,
                 dtype: torch.dtype = torch.float32) -> List[int]:
    """``n_new`` tokens, each the argmax of the last position's logits of the whole sequence so far."""
    seq, out = list(prompt), []
    for _ in range(n_new):
        tok = int(plain_forward(weights, config, seq, dtype)[-1].argmax())
        out.append(tok)
        seq.append(tok)
    return out


# --------------------------------------------------------------------- weights
def plain_weights(config: Mapping, seed: int, stored: torch.dtype = torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors of a configuration, by the names of the checkpoint, with the values that ``stored`` can hold
    (as float32)."""
    g = torch.Generator().manual_seed(seed)
    D, V, S = config["width"], config["vocab"], int(config.get("streams", 1))
    w: Dict[str, torch.Tensor] = {}

    def mat(name, rows, cols, std=None):
        w[name] = torch.randn(rows, cols, generator=g) * (std if std is not None else cols ** -0.5)

    def vec(name, n, mean=0.0, std=0.1):
        w[name] = mean + std * torch.randn(n, generator=g)

    mat("embed", V, D, 1.0)
    vec("final.norm", D, 1.0)
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}"
        vec(f"{p}.norm1", D, 1.0)
        subs = ["hc1"]
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(f"{p}.mix.q", H * 2 * d, D)
            if m.get("kv_from") is None:
                mat(f"{p}.mix.k", G * 2 * d, D)
                mat(f"{p}.mix.v", G * e, D)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                vec(f"{p}.mix.{n}", d, 0.0, 0.3)
            mat(f"{p}.mix.o", D, H * e)
        else:
            H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            mat(f"{p}.mix.q", H * (d + r), D)
            mat(f"{p}.mix.dkv", R + r, D)
            vec(f"{p}.mix.dkv.norm", R, 1.0)
            mat(f"{p}.mix.uk", H * d, R)
            mat(f"{p}.mix.uv", H * e, R)
            vec(f"{p}.mix.sink", H, 0.0, 1.0)
            mat(f"{p}.mix.o", D, H * e)
        mlp = layer.get("mlp")
        if mlp is not None:
            subs.append("hc2")
            vec(f"{p}.norm2", D, 1.0)
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            mat(f"{p}.mlp.router", E, D, 0.5 * D ** -0.5 * 3)
            vec(f"{p}.mlp.correction", E, 0.0, 0.05)
            for e_ in range(E):
                mat(f"{p}.mlp.e{e_}.gate", ff, D, 2 * D ** -0.5)
                mat(f"{p}.mlp.e{e_}.up", ff, D, 2 * D ** -0.5)
                mat(f"{p}.mlp.e{e_}.down", D, ff)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                mat(f"{p}.mlp.shared.gate", sf, D, 2 * D ** -0.5)
                mat(f"{p}.mlp.shared.up", sf, D, 2 * D ** -0.5)
                mat(f"{p}.mlp.shared.down", D, sf)
                mat(f"{p}.mlp.shared.sg", 1, D)
        for q in subs:
            vec(f"{p}.{q}.in", S, 1.0 / S, 0.2)
            vec(f"{p}.{q}.out", S, 1.0, 0.3)
            w[f"{p}.{q}.mix"] = torch.eye(S) + 0.2 * torch.randn(S, S, generator=g)
    return {k: v.to(stored).float() for k, v in w.items()}


# ---------------------------------------------------------------- configurations
def _moe(experts, top, ff, limit, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def _diff(heads, kv, dim, vdim, rot, block, diff, base=5000.0, kv_from=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "diff": diff,
         "rot": {"base": base, "dims": rot}}
    if block:
        m["mask"] = {"size": block}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _latent(heads, dim, rot, vdim, rank, base=300.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "scale": (dim + rot) ** -0.5,
            "rot": {"base": base, "dims": rot}}


# both mixers, a layer on another's keys with a block size of its own, a layer without feed-forward, two streams
PAIR = {"architecture": "Sodotar", "width": 64, "vocab": 96, "norm": {"eps": 1e-5}, "streams": 2, "logit_scale": 0.5,
        "layers": [
            {"type": "attention", "mixer": _diff(4, 2, 16, 32, 8, 24, 0.3), "mlp": _moe(6, 2, 24, 1.0, (40, 1.5))},
            {"type": "latent_attention", "mixer": _latent(3, 16, 8, 24, 24), "mlp": _moe(5, 2, 32, 2.0, (16, 1.0))},
            {"type": "attention", "mixer": _diff(4, 2, 16, 32, 8, 40, 0.5, kv_from=0), "mlp": None},
            {"type": "latent_attention", "mixer": _latent(2, 8, 16, 40, 40), "mlp": _moe(6, 2, 24, 1.0, (40, 1.5))}]}
# one stream, heads that are no power of two, one head a group, values narrower than keys, every dimension rotated,
# no mask, every expert chosen, widths that are no multiple of 8, no shared expert, logits as they are
ODD = {"architecture": "Sodotar", "width": 72, "vocab": 50, "norm": {"eps": 1e-6}, "streams": 1,
       "layers": [
           {"type": "attention", "mixer": _diff(3, 3, 24, 16, 24, None, 0.8), "mlp": _moe(3, 3, 20, 0.7)},
           {"type": "latent_attention", "mixer": _latent(1, 24, 4, 10, 18), "mlp": _moe(4, 1, 12, 1.2, (20, 0.9))},
           {"type": "attention", "mixer": _diff(6, 2, 8, 8, 2, 7, 0.2), "mlp": _moe(4, 1, 12, 1.2, (20, 0.9))}]}
# four streams; twenty heads on one key head (more than the matrix-core kernels group); blocks of one page's size
WIDE = {"architecture": "Sodotar", "width": 64, "vocab": 80, "norm": {"eps": 1e-5}, "streams": 4, "logit_scale": 1.5,
        "layers": [
            {"type": "attention", "mixer": _diff(20, 1, 8, 16, 4, 16, 0.4), "mlp": _moe(8, 3, 16, 1.5, (24, 2.0))},
            {"type": "attention", "mixer": _diff(20, 1, 8, 16, 4, 64, 0.6, kv_from=0), "mlp": _moe(8, 3, 16, 1.5, (24, 2.0))}]}
ONLY_DIFF = {"architecture": "Sodotar", "width": 48, "vocab": 64, "norm": {"eps": 1e-5}, "streams": 1, "logit_scale": 1.0,
             "layers": [{"type": "attention", "mixer": _diff(2, 1, 16, 16, 8, 32, 0.5), "mlp": None}]}
ONLY_LATENT = {"architecture": "Sodotar", "width": 48, "vocab": 64, "norm": {"eps": 1e-5}, "streams": 1, "logit_scale": 1.0,
               "layers": [{"type": "latent_attention", "mixer": _latent(2, 16, 8, 16, 32), "mlp": None}]}
