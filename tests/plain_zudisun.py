"""A plain, slow Zudisun: whole sequences, no cache, no batching, one function
per mechanism, sharing no code with ``fastgen_amd``.  It is what the engine is
compared with.

The model (notation of this file).  Tokens are embedded.  A layer reads the
residual stream itself and norms what its sublayers give:
``x <- x + n1(mixer(x))`` and, if it has a feed-forward, ``x <- x + n2(ff(x))``,
``n`` an RMS norm with a weight.  Two mixers exist:

* ``mamba1``: a selective scan.  ``W_in x = [u | z]``; ``u`` goes through a causal
  convolution per channel (a few taps, a bias) and SiLU; ``W_x u = [r | B | C]``;
  the step ``d = softplus(W_dt r + b)`` per channel; the state
  ``S[c, n] <- exp(d_c A[c, n]) S[c, n] + d_c u_c B_n`` with ``A = -exp(A_log)``;
  ``y_c = sum_n S[c, n] C_n + D_c u_c``; the output is ``W_o (y * silu(z))``.
* ``attention``: grouped heads without rotation and without softmax.  q and k
  are divided by their root mean square per head; q is multiplied by
  ``1 + coef * ln(floor((p + 1) / every) + 1)`` at position ``p``; the score
  ``q . k * scale`` gets a learned bias by the bucket of the distance; the
  heads' scores are mixed by a matrix; the weight of a visible key is
  ``sigmoid(score + b_h)``, not normalised; values may be blended with the
  values that the first such layer computed for the same token; each head's
  output is multiplied by ``sigmoid`` of a gate of its own.

The feed-forward is dense (``down(relu(gate x + b) * (up x + b)) + b``) or routed:
experts without biases and with SiLU, chosen by ``sigmoid`` scores plus a
correction inside the best groups of neighbours, weighted by the scores alone,
plus a shared expert.

``dtype`` is the precision of matrix products and activations; norms, the
residual stream, scores and weights, routers, the recurrence and all that
enters it but the projections and the convolution stay in float32 (float64 when
the whole run is).
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch


def _hi(x: torch.Tensor) -> torch.Tensor:
    return x if x.dtype == torch.float64 else x.float()


def _mm(x: torch.Tensor, w: torch.Tensor, dtype: torch.dtype, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x W^T (+ b)`` with operands in ``dtype``, summed in the high precision, rounded once to ``dtype``."""
    y = _hi(x.to(dtype)) @ _hi(w.to(dtype)).T
    if bias is not None:
        y = y + _hi(bias)
    return y.to(dtype)


# ------------------------------------------------------------------ mechanisms
def plain_rms(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * w`` over the last axis (eps inside the root)."""
    x = _hi(x)
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * _hi(w)


def plain_silu(z: torch.Tensor) -> torch.Tensor:
    z = _hi(z)
    return z * torch.sigmoid(z)


def plain_gated_ff(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, dtype: torch.dtype, act: str,
                   biases: bool) -> torch.Tensor:
    """``down(act(gate x) * (up x))``; ``p`` is the tensors' prefix; with ``biases`` each projection has one."""
    b = (lambda n: w[f"{p}.{n}.b"]) if biases else (lambda n: None)
    g, u = _hi(_mm(x, w[f"{p}.gate"], dtype, b("gate"))), _hi(_mm(x, w[f"{p}.up"], dtype, b("up")))
    a = torch.relu(g) if act == "relu" else plain_silu(g)
    return _mm((a * u).to(dtype), w[f"{p}.down"], dtype, b("down"))


def plain_bucket(n: int, rows: int, far: float) -> int:
    """The row of a distance table of ``rows`` rows for distance ``n >= 0``: one row a distance below
    ``rows / 2``, then logarithmic steps that reach the last row at distance ``far``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def plain_query_temperature(pos: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    return 1.0 + coef * torch.log(torch.floor((pos.double() + 1) / every) + 1.0)


def plain_sigmoid_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, rel: torch.Tensor,
                            far: float, talk: torch.Tensor, head_bias: torch.Tensor) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, e]`` of one sequence (positions 0..T-1), already normed
    and scaled as the design says.  Returns ``[T, H, e]``."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    q, k, v = _hi(q), _hi(k), _hi(v)
    s = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, dim=1)) * scale
    rows = rel.shape[0]
    idx = torch.tensor([[plain_bucket(i - j, rows, far) if j <= i else 0 for j in range(T)] for i in range(T)])
    s = s + _hi(rel)[idx].permute(2, 0, 1)
    s = torch.einsum("hg,gij->hij", talk.to(s.dtype), s) + _hi(head_bias)[:, None, None]
    wgt = torch.sigmoid(s) * torch.tril(torch.ones(T, T, dtype=s.dtype))
    return torch.einsum("hij,jhe->ihe", wgt, v.repeat_interleave(rep, dim=1))


def plain_attention_mixer(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                          dtype: torch.dtype, shared: Dict) -> torch.Tensor:
    """The whole attention mixer on one sequence ``x [T, width]``.  ``shared``: what layers hand on (the first
    value-mixing layer's values)."""
    T = x.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = plain_rms(_mm(x, w[f"{p}.q"], dtype).view(T, H, d), None, eps)
    k = plain_rms(_mm(x, w[f"{p}.k"], dtype).view(T, G, d), None, eps)
    v = _hi(_mm(x, w[f"{p}.v"], dtype)).view(T, G, e)
    q = q * plain_query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"]).to(q.dtype)[:, None, None]
    if m.get("v_mix"):
        if "v_first" in shared:
            lam = _hi(w[f"{p}.vmix"])
            v = (1 - lam) * v + lam * shared["v_first"]
        else:
            shared["v_first"] = v
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    o = plain_sigmoid_attention(q, k, v, m["scale"], w[f"{p}.rel"], m["bias_max"], w[f"{p}.talk"], w[f"{p}.pb"])
    gate = torch.sigmoid(_hi(_mm(x, w[f"{p}.g"], dtype)))  # [T, H]
    o = (o * gate[:, :, None]).to(dtype).reshape(T, H * e)
    return _mm(o, w[f"{p}.o"], dtype)


def plain_causal_conv(u: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``u [T, C]``, ``taps [C, K]`` (the last column meets the current token), zeros before the start."""
    T, C = u.shape
    K = taps.shape[1]
    u, taps = _hi(u), _hi(taps)
    padded = torch.cat([u.new_zeros(K - 1, C), u])
    out = _hi(bias)[None, :].expand(T, C).clone()
    for j in range(K):
        out = out + padded[j:j + T] * taps[:, j][None, :]
    return out


def plain_selective_scan(u: torch.Tensor, step: torch.Tensor, a: torch.Tensor, b: torch.Tensor, c: torch.Tensor,
                         skip: torch.Tensor) -> torch.Tensor:
    """``u, step [T, C]``, ``a [C, N]``, ``b, c [T, N]``, ``skip [C]``: the recurrence token by token."""
    T, C = u.shape
    u, step, a, b, c = _hi(u), _hi(step), _hi(a), _hi(b), _hi(c)
    state = u.new_zeros(C, a.shape[1])
    ys = []
    for t in range(T):
        state = torch.exp(step[t][:, None] * a) * state + (step[t] * u[t])[:, None] * b[t][None, :]
        ys.append(state @ c[t] + _hi(skip) * u[t])
    return torch.stack(ys)


def plain_mamba_mixer(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, dtype: torch.dtype) -> torch.Tensor:
    C, N, R = m["inner"], m["state"], m["dt_rank"]
    uz = _mm(x, w[f"{p}.in"], dtype)
    u, z = uz[:, :C], uz[:, C:]
    u = plain_silu(plain_causal_conv(u, w[f"{p}.conv"], w[f"{p}.conv.b"]).to(dtype)).to(dtype)
    rbc = _mm(u, w[f"{p}.x"], dtype)
    r, b, c = rbc[:, :R], rbc[:, R:R + N], rbc[:, R + N:]
    step = torch.nn.functional.softplus(_hi(_mm(r, w[f"{p}.dt"], dtype)) + _hi(w[f"{p}.dt.b"]))
    a = -torch.exp(_hi(w[f"{p}.A_log"]))
    y = plain_selective_scan(u, step, a, b, c, w[f"{p}.D"])
    return _mm((y * plain_silu(z)).to(dtype), w[f"{p}.o"], dtype)


def plain_route(x: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int,
                scale: float):
    """Per row of ``x [T, width]``: the chosen experts ``[T, top]`` and their weights."""
    s = torch.sigmoid(_hi(x) @ router.to(_hi(x).dtype).T)
    choice = s + _hi(correction)
    T, E = s.shape
    per = E // groups
    by_group = choice.view(T, groups, per)
    group_score = by_group.topk(min(2, per), dim=-1).values.sum(-1)
    kept = group_score.topk(keep, dim=-1).indices
    mask = torch.zeros(T, groups, dtype=torch.bool)
    mask.scatter_(1, kept, True)
    masked = torch.where(mask[:, :, None].expand(T, groups, per).reshape(T, E), choice, torch.full_like(choice, -math.inf))
    chosen = masked.topk(top, dim=-1).indices
    wgt = s.gather(1, chosen)
    wgt = wgt / (wgt.sum(-1, keepdim=True) + 1e-20) * scale
    return chosen, wgt


def plain_routed_ff(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, mlp: Mapping, dtype: torch.dtype) -> torch.Tensor:
    r = mlp["router"]
    chosen, wgt = plain_route(x.to(dtype), w[f"{p}.router"], w[f"{p}.correction"], r["top"], r["groups"]["count"],
                              r["groups"]["keep"], r["scale"])
    out = _hi(x).new_zeros(x.shape)
    for t in range(x.shape[0]):
        for j in range(r["top"]):
            e = int(chosen[t, j])
            out[t] += wgt[t, j] * _hi(plain_gated_ff(x[t:t + 1], w, f"{p}.e{e}", dtype, "silu", False))[0]
    if mlp.get("shared"):
        out = out + _hi(plain_gated_ff(x, w, f"{p}.shared", dtype, "silu", False))
    return out


# ------------------------------------------------------------------ the model
def plain_zudisun_forward(config: Mapping, w: Mapping[str, torch.Tensor], tokens: List[int],
                          dtype: torch.dtype = torch.float32, layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence.  ``layers_out``: a list that receives the stream after every layer."""
    eps = config["norm"]["eps"]
    hi = torch.float64 if dtype == torch.float64 else torch.float32
    x = w["embed"][torch.tensor(tokens)].to(hi)
    shared: Dict = {}
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}"
        if layer["type"] == "attention":
            y = plain_attention_mixer(x, w, f"{p}.mix", layer["mixer"], eps, dtype, shared)
        elif layer["type"] == "mamba1":
            y = plain_mamba_mixer(x, w, f"{p}.mix", layer["mixer"], dtype)
        else:
            raise ValueError(layer["type"])
        x = x + plain_rms(y, w[f"{p}.norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                y = plain_gated_ff(x, w, f"{p}.mlp", dtype, "relu", True)
            else:
                y = plain_routed_ff(x, w, f"{p}.mlp", mlp, dtype)
            x = x + plain_rms(y, w[f"{p}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return _hi(_mm(plain_rms(x, w["final.norm"], eps), w["head"], dtype))


def plain_zudisun_greedy(config: Mapping, w: Mapping[str, torch.Tensor], prompt: List[int], n_new: int,
                         dtype: torch.dtype = torch.float32) -> List[int]:
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(int(plain_zudisun_forward(config, w, seq, dtype)[-1].argmax()))
    return seq[len(prompt):]


# ------------------------------------------------------------------ shapes, weights, configurations
def plain_zudisun_shapes(config: Mapping, bias_rows: int = 32) -> Dict[str, tuple]:
    """The tensors of a model: name -> shape.  ``bias_rows``: rows of every distance table (a mixer's own
    ``bias_rows`` key, if it has one, goes first)."""
    W, out = config["width"], {}
    out["embed"] = (config["vocab"], W)
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}", layer["mixer"]
        out[f"{p}.norm1"] = (W,)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({f"{p}.mix.q": (H * d, W), f"{p}.mix.k": (G * d, W), f"{p}.mix.v": (G * e, W),
                        f"{p}.mix.rel": (m.get("bias_rows", bias_rows), H), f"{p}.mix.talk": (H, H), f"{p}.mix.pb": (H,),
                        f"{p}.mix.g": (H, W), f"{p}.mix.o": (W, H * e)})
            if m.get("v_mix"):
                out[f"{p}.mix.vmix"] = ()
        else:
            C, N, R, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            out.update({f"{p}.mix.in": (2 * C, W), f"{p}.mix.conv": (C, K), f"{p}.mix.conv.b": (C,),
                        f"{p}.mix.x": (R + 2 * N, C), f"{p}.mix.dt": (C, R), f"{p}.mix.dt.b": (C,),
                        f"{p}.mix.A_log": (C, N), f"{p}.mix.D": (C,), f"{p}.mix.o": (W, C)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[f"{p}.norm2"] = (W,)
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            out.update({f"{p}.mlp.gate": (F, W), f"{p}.mlp.gate.b": (F,), f"{p}.mlp.up": (F, W), f"{p}.mlp.up.b": (F,),
                        f"{p}.mlp.down": (W, F), f"{p}.mlp.down.b": (W,)})
        else:
            F, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            for e_ in range(E):
                out.update({f"{p}.mlp.e{e_}.gate": (F, W), f"{p}.mlp.e{e_}.up": (F, W), f"{p}.mlp.e{e_}.down": (W, F)})
            out.update({f"{p}.mlp.router": (E, W), f"{p}.mlp.correction": (E,)})
            if mlp.get("shared"):
                S = mlp["shared"]["ff"]
                out.update({f"{p}.mlp.shared.gate": (S, W), f"{p}.mlp.shared.up": (S, W), f"{p}.mlp.shared.down": (W, S)})
    out["final.norm"] = (W,)
    out["head"] = (config["vocab"], W)
    return out


def plain_zudisun_weights(config: Mapping, seed: int) -> Dict[str, torch.Tensor]:
    """Random weights, representable in bfloat16, large enough that every mechanism moves the logits."""
    g = torch.Generator().manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    for name, shape in plain_zudisun_shapes(config).items():
        r = lambda std: std * torch.randn(shape, generator=g)
        if name.endswith(("norm1", "norm2", "norm")):
            t = 1.0 + r(0.2)
        elif name.endswith(".vmix"):
            t = 0.35 + r(0.1)
        elif name.endswith(".rel"):
            t = r(0.7)
        elif name.endswith(".talk"):
            t = torch.eye(shape[0]) + r(0.25)
        elif name.endswith(".pb"):
            t = -2.0 + r(0.7)  # sums over hundreds of keys stay moderate
        elif name.endswith(".A_log"):
            t = torch.log(torch.arange(1, shape[1] + 1, dtype=torch.float32))[None, :].expand(shape) + r(0.2)
        elif name.endswith(".dt.b"):
            t = -2.0 + r(1.0)
        elif name.endswith(".D"):
            t = 1.0 + r(0.3)
        elif name.endswith(".correction"):
            t = r(0.3)
        elif name.endswith(".conv"):
            t = r(0.5)
        elif name.endswith(".b"):
            t = r(0.3)
        elif name.endswith(".router"):
            t = r(4.0 / math.sqrt(shape[-1]))
        elif name == "embed":
            t = r(1.0)
        else:
            t = r(1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16).float()
    return out


def _sig(H, G, d, e, every=16, coef=0.5, far=40, v_mix=False, rows=None):
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": e, "scale": d ** -0.5, "q_temp": {"coef": coef, "every": every},
         "bias_max": far, "v_mix": v_mix}
    if rows is not None:
        m["bias_rows"] = rows
    return m


def _scan(C, N, R, K):
    return {"inner": C, "state": N, "dt_rank": R, "conv": K}


def _moe(E, top, F, groups=1, keep=1, scale=1.0, shared=None):
    return {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": top, "scale": scale,
                                                             "groups": {"count": groups, "keep": keep}},
            "shared": None if shared is None else {"ff": shared}}


def _zconfig(width, vocab, layers, eps=1e-5):
    return {"architecture": "Zudisun", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}


# both mixers, both feed-forwards, a layer without one; values mixed over three layers; tables of 12 rows
PAIR = _zconfig(64, 97, [
    {"type": "mamba1", "mixer": _scan(96, 8, 6, 4), "mlp": _moe(6, 2, 40, groups=3, keep=2, scale=2.0, shared=48)},
    {"type": "attention", "mixer": _sig(4, 2, 32, 16, far=30, v_mix=True, rows=12), "mlp": {"kind": "dense", "ff": 96}},
    {"type": "attention", "mixer": _sig(2, 2, 16, 16, every=5, coef=1.5, far=100, v_mix=True, rows=12), "mlp": None},
    {"type": "mamba1", "mixer": _scan(80, 16, 4, 2), "mlp": {"kind": "dense", "ff": 72}},
    {"type": "attention", "mixer": _sig(6, 2, 16, 16, every=64, far=13, v_mix=True, rows=12), "mlp": _moe(4, 1, 56)},
])
# one layer of a kind each, for tests of a mechanism inside the engine
ONLY_SIGMOID = _zconfig(48, 61, [{"type": "attention", "mixer": _sig(2, 1, 16, 24, every=7, far=50, rows=16),
                                  "mlp": {"kind": "dense", "ff": 56}}])
ONLY_SCAN = _zconfig(48, 61, [{"type": "mamba1", "mixer": _scan(64, 12, 5, 3), "mlp": None}])
# sizes that are no multiples of 8 or 16, head counts that are no powers of two, one kv head for all and one a
# head, values wider than keys, one tap and many taps, a state of one and of many values, a step rank of one,
# tables with an odd number of rows, a far distance beyond every prompt and one just past half of the table,
# a temperature that changes at every position and one that never does, every expert chosen, a group an
# expert, no shared expert, groups of which all stay, a mixing layer between layers that do not mix
ODD = _zconfig(100, 101, [
    {"type": "attention", "mixer": _sig(5, 5, 20, 12, every=1, coef=0.25, far=1000.0, rows=9), "mlp": _moe(3, 3, 36, scale=0.5)},
    {"type": "mamba1", "mixer": _scan(70, 1, 1, 1), "mlp": None},
    {"type": "attention", "mixer": _sig(7, 1, 10, 26, every=100000, far=5, v_mix=True, rows=7), "mlp": {"kind": "dense", "ff": 36}},
    {"type": "mamba1", "mixer": _scan(36, 37, 9, 9), "mlp": _moe(8, 2, 20, groups=8, keep=3, shared=28)},
    {"type": "attention", "mixer": _sig(3, 1, 10, 26, every=3, coef=2.0, far=64.5, v_mix=True, rows=7), "mlp": _moe(6, 4, 24, groups=2, keep=2)},
    {"type": "attention", "mixer": _sig(34, 2, 8, 8, far=33, rows=64), "mlp": None},
], eps=1e-4)
# recurrent layers alone: a model without a cache of keys
NO_CACHE = _zconfig(56, 83, [
    {"type": "mamba1", "mixer": _scan(48, 4, 3, 5), "mlp": {"kind": "dense", "ff": 64}},
    {"type": "mamba1", "mixer": _scan(112, 20, 8, 2), "mlp": _moe(5, 2, 32, shared=16)},
])
