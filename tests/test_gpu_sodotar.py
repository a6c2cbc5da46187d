"""Sodotar on the GPU against the plain implementation (``tests/plain_sodotar.py``) and the kernels' plain
twins: each new kernel alone, then whole models of several shapes under every way of cutting requests into
steps, with small pools so that pages and slots change hands, in float32 (strict) and bfloat16."""

from __future__ import annotations

import copy
from typing import Dict, List

import pytest
import torch

import traces
from helpers import make_runner, run_trace, save_model_folder
from plain_sodotar import (ODD, ONLY_DIFF, ONLY_LATENT, PAIR, WIDE, plain_block_mask, plain_forward, plain_greedy,
                           plain_weights)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CONFIGS = {"pair": PAIR, "odd": ODD, "wide": WIDE, "only_diff": ONLY_DIFF, "only_latent": ONLY_LATENT}


def _tokens(config, lengths: Dict[str, int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {r: torch.randint(0, config["vocab"], (n,), generator=g).tolist() for r, n in lengths.items()}


def _close(got, want, dtype, what=""):
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), msg=lambda m: f"{what}: {m}", **tol)


def _routed(config) -> bool:
    return any(l.get("mlp") is not None for l in config["layers"])


def _close_to_plain(got, want, noise, dtype, what, routed):
    """The engine against the plain run ``want`` with the plain run at the engine's precision (``noise``) as the
    yardstick: float32 (``want``: the float64 run) three times that run's worst error; bfloat16 (``want``: the
    float32 run) twice, of which nine tenths may be used.  bfloat16 with routed experts: a choice of experts within
    rounding of a tie may fall the other way than in the plain bfloat16 run, so nine in ten positions keep to the
    tolerance and none is off by more than such a choice can explain."""
    level = max(float((noise[r].double() - want[r].double()).abs().max()) for r in want)
    n_over = n_all = 0
    for rid, w in want.items():
        g = got[rid]
        assert g.shape == w.shape and torch.isfinite(g).all(), f"{what} {rid}"
        scale = float(w.abs().max())
        err = (g.double() - w.double()).abs().amax(-1)
        tol = 3.0 * level + 1e-6 * scale if dtype == torch.float32 else 0.9 * (2.0 * level + 1e-3 * scale)
        over = (err > tol).nonzero().flatten().tolist()
        if dtype == torch.bfloat16 and routed:
            n_over, n_all = n_over + len(over), n_all + len(err)
            assert float(err.max()) <= scale, f"{what} {rid}: {float(err.max()):.3e}"
        else:
            assert not over, f"{what} {rid}: positions {over[:8]} over {tol:.3e}, worst {float(err.max()):.3e}"
    assert n_over <= 0.1 * n_all, f"{what}: {n_over} of {n_all} positions over the tolerance"


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,T,D", [(1, 5, 40), (3, 7, 200), (4, 70, 1000), (8, 3, 2304), (5, 4, 1536), (2, 6, 42), (3, 5, 4096), (7, 9, 1024), (11, 3, 512), (16, 2, 100)])
def test_streams_step_and_spread(dtype, S, T, D):
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(S * T + D)
    h = torch.randn(T, D, generator=g)
    x = ops.streams_spread(h.to(DEV), S)
    assert torch.equal(x.cpu(), twins.streams_spread(h, S))
    x = torch.randn(S, T, D, generator=g)
    w = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    a, b, M = torch.randn(S, generator=g), torch.randn(S, generator=g), torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)
    rows = torch.tensor([T - 1, 0, T - 1], dtype=torch.int32)
    for delta in (torch.randn(T, D, generator=g).to(dtype), torch.randn(3, T, D, generator=g), None):
        upd_c = None if delta is None else twins_update(delta, M, b)
        upd_g = None if delta is None else ops.StreamUpdate(delta.to(DEV), M.to(DEV).contiguous(), b.to(DEV))
        # gathered rows leave the streams alone
        xg = x.clone().to(DEV)
        out_c, out_g = torch.empty(3, D, dtype=dtype), torch.empty(3, D, dtype=dtype, device=DEV)
        twins.streams_step(x.clone(), upd_c, None, w, 1e-5, out_c, rows)
        ops.streams_step(xg, upd_g, None, w.to(DEV), 1e-5, out_g, rows.to(DEV))
        assert torch.equal(xg.cpu(), x)
        _close(out_g, out_c, dtype, "gathered")
        # all rows: the streams are updated in place, u is what the norm reads
        xc = x.clone()
        out_c, out_g = torch.empty(T, D, dtype=dtype), torch.empty(T, D, dtype=dtype, device=DEV)
        u_c, u_g = torch.empty(T, D), torch.empty(T, D, device=DEV)
        twins.streams_step(xc, upd_c, a, w, 1e-5, out_c, None, u_c)
        ops.streams_step(xg, upd_g, a.to(DEV), w.to(DEV), 1e-5, out_g, None, u_g)
        _close(xg, xc, torch.float32, "streams")
        _close(u_g, u_c, torch.float32, "sum")
        _close(out_g, out_c, dtype, "normed")


def twins_update(delta, M, b):
    from fastgen_amd.kernels import ops

    return ops.StreamUpdate(delta, M.contiguous(), b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,group,hw,e", [(4, 2, 32, 32), (3, 1, 32, 10), (20, 20, 16, 16), (6, 3, 96, 80)])
def test_head_diff_norm(dtype, H, group, hw, e):
    from fastgen_amd.kernels import ops, twins

    T = 9
    att = torch.randn(T, 2 * H * hw, generator=torch.Generator().manual_seed(H + e)).to(dtype)
    out_c, out_g = torch.zeros(T, H * e, dtype=dtype), torch.zeros(T, H * e, dtype=dtype, device=DEV)
    twins.head_diff_norm(att, hw, out_c, H, group, e, 0.37, 1e-5, 0.6)
    ops.head_diff_norm(att.to(DEV), hw, out_g, H, group, e, 0.37, 1e-5, 0.6)
    _close(out_g, out_c, dtype, "head_diff_norm")
    # written from the formula: head h's maps lie at (h // group) * 2 * group + h % group and `group` heads on
    a = att.float().view(T, 2 * H, hw)
    for h in (0, H - 1):
        i = (h // group) * 2 * group + h % group
        o = a[:, i, :e] - 0.37 * a[:, i + group, :e]
        want = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5) * 0.6
        _close(out_c[:, h * e : (h + 1) * e], want.to(dtype), dtype, f"twin, head {h}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routing_by_a_softmax_over_all_experts_with_a_gate_row(dtype):
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(4)
    for T, D, E, top in ((5, 64, 6, 2), (70, 40, 3, 3), (9, 72, 16, 1)):
        x = torch.randn(T, D, generator=g).to(dtype)
        router, corr = torch.randn(E + 1, D, generator=g) * 0.3, torch.randn(E, generator=g) * 0.2
        ci, cw, ce = twins.moe_route(x, router, None, top, False, corr, 1, 1, 1.0, True, 1)
        gi, gw, ge = ops.moe_route(x.to(DEV), router.to(DEV), None, top, False, corr.to(DEV), 1, 1, 1.0, True, 1)
        assert torch.equal(gi.cpu(), ci)
        _close(gw, cw, torch.float32, "weights")
        _close(ge, ce, torch.float32, "gate logits")
        # from the formula
        s = torch.softmax(x.float() @ router[:E].T, -1)
        pick = torch.sort(s + corr, dim=-1, descending=True, stable=True).indices[:, :top]
        assert torch.equal(ci.long(), pick)
        ws = s.gather(1, pick)
        _close(cw, ws / ws.sum(-1, keepdim=True), torch.float32, "twin weights")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D,F,E,top", [(6, 64, 24, 5, 2), (300, 64, 32, 4, 2), (40, 72, 20, 3, 3)])
def test_experts_with_the_limited_activation_and_a_gated_shared_expert(dtype, T, D, F, E, top):
    from fastgen_amd.kernels import ops, twins
    from fastgen_amd.parts.moe import MoE
    from fastgen_amd.config import PartSpec

    g = torch.Generator().manual_seed(T + F)
    spec = PartSpec("moe", "m", dict(dim=D, hidden_dim=F, n_experts=E, top=top, router_bias=False, scoring="softmax_all",
                                     correction=True, activation="limited", limit=0.8, alpha=1.702, shared_hidden_dim=16,
                                     shared_activation="limited", shared_limit=0.5, shared_gate=True))
    part = MoE(spec)
    tensors = {s.name: (torch.randn(s.shape, generator=g) * (0.3 if "router" in s.name or "gate" in s.name else 0.15)).to(dtype).float()
               for s in part.tensor_specs()}
    part.load(tensors, dtype, DEV)
    x = torch.randn(T, D, generator=g).to(dtype)
    got = part.forward(x.to(DEV))[0].cpu()
    # the plain formula
    from plain_sodotar import plain_moe
    w = {"p.router": tensors["m.router.weight"], "p.correction": tensors["m.correction"], "p.shared.sg": tensors["m.shared_gate.weight"]}
    for e in range(E):
        for n in ("gate", "up", "down"):
            w[f"p.e{e}.{n}"] = tensors[f"m.experts.{e}.{n}_proj.weight"]
    for n in ("gate", "up", "down"):
        w[f"p.shared.{n}"] = tensors[f"m.shared.{n}_proj.weight"]
    mlp = {"router": {"experts": E, "top": top}, "expert": {"limit": 0.8}, "shared": {"limit": 0.5}}
    want = plain_moe(x, w, "p", mlp, dtype)
    if dtype == torch.float32:
        _close(got, want, dtype, "experts")
    else:  # a choice within rounding of a tie may differ
        bad = ((got - want).abs().amax(-1) > 0.03 * float(want.abs().max())).sum()
        assert int(bad) <= 0.1 * T
    # the activation kernel alone against its twin
    gu = torch.randn(T, 2 * 32, generator=g)
    _close(ops.gated_mul(gu.to(DEV), None, "limited", dtype, None, 0.7, 1.702), twins.gated_mul(gu, None, "limited", dtype, None, 0.7, 1.702),
           dtype, "gated_mul")


@pytest.mark.parametrize("dtype,P", [(torch.float32, 16), (torch.bfloat16, 16), (torch.bfloat16, 64)])
@pytest.mark.parametrize("block", [5, 16, 64, 100])
def test_attention_over_blocks_of_positions(dtype, P, block):
    """The engine's attention kernels with a mask of blocks (``window`` < 0) against the twin: a prompt in one
    step (the general kernel, or tiles on the matrix cores), and its last tokens alone (split keys)."""
    from fastgen_amd.cache.layout import pack_k, pack_v
    from fastgen_amd.kernels import ops, twins

    H, KV, hd, n = 4, 2, 32, 230
    g = torch.Generator().manual_seed(block)
    q = torch.randn(n, H * hd, generator=g).to(dtype)
    k, v = torch.randn(n, KV, hd, generator=g).to(dtype), torch.randn(n, KV, hd, generator=g).to(dtype)
    n_pages = -(-n // P)
    pad = n_pages * P - n
    kn = torch.cat([k, torch.zeros(pad, KV, hd, dtype=dtype)]).view(n_pages, P, KV, hd).permute(0, 2, 1, 3).contiguous()
    vn = torch.cat([v, torch.zeros(pad, KV, hd, dtype=dtype)]).view(n_pages, P, KV, hd).permute(0, 2, 1, 3).contiguous()
    kp, vp = pack_k(kn), pack_v(vn)
    bt = torch.arange(n_pages, dtype=torch.int32)[None]
    seq, pos = torch.zeros(n, dtype=torch.int32), torch.arange(n, dtype=torch.int32)
    want = torch.empty(n, H * hd, dtype=dtype)
    twins.paged_attention_general(q, want, kp, vp, bt, seq, pos, H, 0.2, -block)
    # the twin against the formula
    vis = plain_block_mask(n, block)
    s = torch.einsum("thd,jhd->htj", q.float().view(n, H, hd), k.float().repeat_interleave(H // KV, 1)) * 0.2
    a = torch.softmax(s.masked_fill(~vis[None], float("-inf")), -1)
    plain = torch.einsum("htj,jhd->thd", a, v.float().repeat_interleave(H // KV, 1)).reshape(n, -1)
    _close(want, plain.to(dtype), dtype, "twin")
    got = torch.empty(n, H * hd, dtype=dtype, device=DEV)
    ops.paged_attention_general(q.to(DEV), got, kp.to(DEV), vp.to(DEV), bt.to(DEV), seq.to(DEV), pos.to(DEV), H, 0.2, -block)
    _close(got, want, dtype, "general kernel")
    if dtype == torch.bfloat16:
        per_tile = max(1, ops.attention_tile_rows(hd) // (H // KV))
        big = torch.tensor([[0, i, min(per_tile, n - i), i] for i in range(0, n, per_tile)], dtype=torch.int32, device=DEV)
        tiles = torch.empty_like(got)
        ops.paged_attention_mfma(q.to(DEV), tiles, kp.to(DEV), vp.to(DEV), bt.to(DEV), None, big, H, 0.2, -block)
        _close(tiles, want, dtype, "tiles")
        for first in (n - 1, n - 3, block * (n // block), block * (n // block) - 1):
            m, per = n - first, 16 // (H // KV)  # items of at most 16 rows (tokens times the heads of a group)
            small = torch.tensor([[0, i, min(per, m - i), first + i] for i in range(0, m, per)], dtype=torch.int32, device=DEV)
            cut = torch.empty(m, H * hd, dtype=dtype, device=DEV)
            ops.paged_attention_mfma(q[first:].to(DEV), cut, kp.to(DEV), vp.to(DEV), bt.to(DEV), small, None, H, 0.2, -block)
            _close(cut, want[first:], dtype, f"split keys from {first}")


# ----------------------------------------------------------------- whole models
LENGTHS = {"a": 150, "b": 37, "c": 2, "d": 1, "e": 70, "f": 19}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        weights = plain_weights(config, seed=len(name))
        folder = save_model_folder(tmp_path_factory.mktemp(name), config, weights)
        toks = _tokens(config, LENGTHS, seed=7)
        out[name] = (config, weights, folder, toks, {r: plain_forward(weights, config, t) for r, t in toks.items()})
    return out


@pytest.fixture(scope="module")
def exact(cases):
    """The float64 runs of the same requests: what float32 results are measured against where sums are long."""
    return {name: {r: plain_forward(c[1], c[0], t, torch.float64) for r, t in c[3].items()} for name, c in cases.items()}


def _all_traces(lengths):
    return {"whole": traces.whole(lengths), "tail": traces.tail(lengths, 60), "chunks": traces.chunks(lengths),
            "pairs": traces.chunks(lengths, sizes=(2, 3, 2, 5)),
            "mixed": traces.mixed(lengths, seed=3), "mixed2": traces.mixed(lengths, max_live=3, seed=11, budget=23)}


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_float32_every_cut_batch_and_reuse(cases, exact, name):
    """Whole prompts, prompts then single tokens, portions down to two tokens and one, mixed batches of unequal
    requests: the same logits as the plain run whatever the cut.  Pages of 16 tokens and a pool that holds the
    live requests only: pages and slots are used again."""
    config, weights, folder, toks, want = cases[name]
    runner = make_runner(folder, torch.float32, page_size=16, max_tokens=304, max_requests=4)
    first = None
    for kind, tr in _all_traces(LENGTHS).items():
        got = run_trace(runner, tr, toks)
        _close_to_plain(got, exact[name], want, torch.float32, f"sodotar {name} {kind}", _routed(config))
        if first is None:
            first = got
        else:
            for r in got:
                scale = float(first[r].abs().max())
                assert float((got[r] - first[r]).abs().max()) <= 1e-5 * scale, f"{name} {kind}: request {r} depends on the cut"
        assert all(runner.cache.free_pages(g) == 304 // 16 for g in range(runner.cache.n_groups))
        assert runner.cache.free_slots() == 4


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_bfloat16_every_cut_batch_and_reuse(cases, name):
    config, weights, folder, toks, want = cases[name]
    noise = {r: plain_forward(weights, config, t, torch.bfloat16) for r, t in toks.items()}
    for page, pool in ((16, 304), (64, 768)):  # (pages of 64: whole pages go straight into LDS)
        runner = make_runner(folder, torch.bfloat16, page_size=page, max_tokens=pool, max_requests=4)
        for kind, tr in _all_traces(LENGTHS).items():
            _close_to_plain(run_trace(runner, tr, toks), want, noise, torch.bfloat16,
                            f"sodotar {name} {kind} bfloat16, pages of {page}", _routed(config))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_streams_after_every_layer(cases, dtype):
    """The sum of the residual streams after each layer, read from the engine behind every layer's arrangement."""
    from fastgen_amd.engine import Model, ModelRunner, StepEntry
    from fastgen_amd.kernels import ops

    config, weights, folder, toks, _ = cases["pair"]
    want: list = []
    plain_forward(weights, config, toks["b"], dtype, want)
    model = Model.from_folder(folder, dtype, DEV)
    seen = []
    for block in model.parts.blocks:
        def wrap(keep=block.forward):
            def forward(h, pending, ctx, store):
                out = keep(h, pending, ctx, store)
                n = h.shape[1]
                u = torch.empty((n, h.shape[2]), dtype=torch.float32, device=h.device)
                ops.streams_step(h, out, None, None, 0.0, None, torch.arange(n, dtype=torch.int32, device=h.device), u)
                seen.append(u.cpu())
                return out
            return forward
        block.forward = wrap()
    runner = ModelRunner(model, page_size=16, max_tokens=64, max_requests=1)
    runner.step([StepEntry("b", toks["b"], [0])])
    assert len(seen) == len(want)
    for i, (g, w) in enumerate(zip(seen, want)):
        tol = 2e-5 if dtype == torch.float32 else 4e-2
        off = ((g - w.float()).abs().amax(-1) > tol * float(w.abs().max())).nonzero().flatten().tolist()
        assert len(off) <= (0 if dtype == torch.float32 else 0.1 * len(toks["b"])), f"after layer {i}: rows {off}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["pair", "odd"])
def test_long_decoding_across_pages_and_blocks(cases, dtype, name):
    """A short prompt, then 290 tokens one by one over many pages and many blocks of the mask (bfloat16: recorded
    steps)."""
    config, weights, folder, _, _ = cases[name]
    toks = _tokens(config, {"z": 300}, seed=5)
    want = {"z": plain_forward(weights, config, toks["z"])}
    runner = make_runner(folder, dtype, page_size=16, max_tokens=304, max_requests=2)
    got = run_trace(runner, traces.tail({"z": 300}, 290), toks)
    if dtype == torch.float32:
        _close_to_plain(got, {"z": plain_forward(weights, config, toks["z"], torch.float64)}, want, dtype,
                        f"sodotar {name} long decoding", True)
    else:
        _close_to_plain(got, want, {"z": plain_forward(weights, config, toks["z"], torch.bfloat16)}, dtype,
                        f"sodotar {name} long decoding bfloat16", True)


@pytest.mark.parametrize("name", ["pair", "wide"])
def test_long_prompts_beside_short_ones(cases, name):
    """Prompts of several hundred tokens in one step, together in one batch, in two steps and in small portions."""
    config, weights, folder, _, _ = cases[name]
    lengths = {"p": 700, "q": 260, "r": 3}
    toks = _tokens(config, lengths, seed=13)
    want = {r: plain_forward(weights, config, t) for r, t in toks.items()}
    exact = {r: plain_forward(weights, config, t, torch.float64) for r, t in toks.items()}
    noise = {r: plain_forward(weights, config, t, torch.bfloat16) for r, t in toks.items()}
    together = [([("p", 0, 700), ("q", 0, 260), ("r", 0, 3)], ["p", "q", "r"])]
    for dtype, page in ((torch.float32, 16), (torch.bfloat16, 16), (torch.bfloat16, 64)):
        runner = make_runner(folder, dtype, page_size=page, max_tokens=1152, max_requests=3)
        for kind, tr in (("whole", traces.whole(lengths)), ("together", together),
                         ("halves", traces.chunks(lengths, sizes=(390, 310))), ("portions", traces.chunks(lengths))):
            got = run_trace(runner, tr, toks)
            if dtype == torch.float32:
                _close_to_plain(got, exact, want, dtype, f"sodotar {name} long {kind}", True)
            else:
                _close_to_plain(got, want, noise, dtype, f"sodotar {name} long {kind} bfloat16", True)


def _sharp(config, weights, factor):
    """Queries scaled up, so that a token's weight lies on few keys and a key that is wrongly seen or missed moves
    the logits by far more than rounding does."""
    w = dict(weights)
    for i in range(len(config["layers"])):
        w[f"l{i}.mix.q"] = w[f"l{i}.mix.q"] * factor
    return w


def test_keys_at_the_edges_of_blocks_and_pages(tmp_path):
    """One layer of differential attention with sharp scores and blocks of 32, 16 (one page) and 21 positions:
    the plain run with a block one position longer or shorter differs by far more than the tolerance at the
    positions behind a block's edge, and the engine agrees with the right one, for whole prompts, portions down to
    two tokens and tokens decoded alone."""
    n = 150
    for block in (32, 16, 21):
        config = copy.deepcopy(ONLY_DIFF)
        config["layers"][0]["mixer"]["mask"]["size"] = block
        w = _sharp(config, plain_weights(config, block), 6.0)
        toks = _tokens(config, {"s": n}, seed=block)
        want = {"s": plain_forward(w, config, toks["s"])}
        for other_size in (block - 1, block + 1):
            other = copy.deepcopy(config)
            other["layers"][0]["mixer"]["mask"]["size"] = other_size
            moved = (plain_forward(w, other, toks["s"]) - want["s"]).abs().amax(-1)
            assert float(moved[block:].max()) > 0.05 * float(want["s"].abs().max()), "the blocks' edges do not decide"
        folder = save_model_folder(tmp_path / f"b{block}", config, w)
        for dtype, page in ((torch.float32, 16), (torch.bfloat16, 16), (torch.bfloat16, 64)):
            runner = make_runner(folder, dtype, page_size=page, max_tokens=256, max_requests=1)
            noise = {"s": plain_forward(w, config, toks["s"], torch.bfloat16 if dtype == torch.bfloat16 else torch.float64)}
            ref = want if dtype == torch.bfloat16 else noise
            for tr in (traces.whole({"s": n}), traces.tail({"s": n}, 100), traces.chunks({"s": n}),
                       traces.chunks({"s": n}, sizes=(2, 3, 2, 5))):
                _close_to_plain(run_trace(runner, tr, toks), ref, noise if dtype == torch.bfloat16 else want, dtype,
                                f"block {block}", False)


def test_a_far_key_and_the_sink(tmp_path):
    """One layer of latent attention with sharp scores: the last tokens of 600 put their weight on keys hundreds of
    positions back (changing the first 40 tokens changes the last logits), and the sink takes a visible share
    (without it the logits differ): whole, in portions, decoded alone, through pages that another request held."""
    config = copy.deepcopy(ONLY_LATENT)
    w = _sharp(config, plain_weights(config, 9), 5.0)
    w["l0.mix.sink"] = torch.tensor([12.0, 14.0])
    n = 600
    toks = _tokens(config, {"other": 70, "s": n}, seed=2)
    want = {r: plain_forward(w, config, t) for r, t in toks.items()}
    scale = float(want["s"].abs().max())
    without = list(toks["s"])
    for i in range(40):
        without[i] = (without[i] + 1) % config["vocab"]
    assert float((plain_forward(w, config, without)[-30:] - want["s"][-30:]).abs().max()) > 0.05 * scale, "no far key counts"
    no_sink = dict(w)
    no_sink["l0.mix.sink"] = torch.tensor([-30.0, -30.0])
    moved = (plain_forward(no_sink, config, toks["s"]) - want["s"]).abs().amax(-1)
    assert float((moved > 0.01 * scale).float().mean()) > 0.5, "the sink does not count"
    folder = save_model_folder(tmp_path / "m", config, w)
    lengths = {"other": 70, "s": n}
    for dtype, page in ((torch.float32, 16), (torch.bfloat16, 64)):
        runner = make_runner(folder, dtype, page_size=page, max_tokens=640, max_requests=1)
        hi = {r: plain_forward(w, config, t, torch.float64 if dtype == torch.float32 else torch.bfloat16) for r, t in toks.items()}
        for tr in (traces.whole(lengths), traces.tail(lengths, 40), traces.chunks(lengths), traces.chunks(lengths, sizes=(2, 3, 2, 64))):
            if dtype == torch.float32:
                _close_to_plain(run_trace(runner, tr, toks), hi, want, dtype, "far key", False)
            else:
                _close_to_plain(run_trace(runner, tr, toks), want, hi, dtype, "far key bfloat16", False)


def test_greedy_generation_through_the_engine(cases):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    config, weights, folder, toks, _ = cases["pair"]
    prompts = [toks["b"], toks["f"], toks["c"], toks["e"][:40], toks["d"]]
    want = [plain_greedy(weights, config, p, 9) for p in prompts]
    engine = Engine.from_folder(folder, torch.float32, DEV, page_size=16, max_tokens=320, max_batch=3, max_step_tokens=24)
    assert engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=9)) == want
    low = Engine.from_folder(folder, torch.bfloat16, DEV, page_size=16, max_tokens=320, max_batch=3, max_step_tokens=24)
    got = low.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=9))
    assert [len(g) for g in got] == [9] * len(prompts)


def test_command_lines(cases, tmp_path):
    """The trace runner and the chat tool take the model by its folder, as they take any other."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    config, weights, folder, toks, want = cases["odd"]
    root = Path(__file__).resolve().parents[1]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks["b"][:20], "want": [19]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks["b"][20:], "want": [0, 16]}], "end": ["x"]}]
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1"]
    got = np.fromfile(out / "1.f32", dtype="<f4").reshape(2, -1)
    assert np.abs(got - want["b"][[20, 36]].numpy()).max() <= 2e-5 * float(want["b"].abs().max())
    chat = subprocess.run([sys.executable, str(root / "bin" / "fgchat"), str(folder), "--prompt-ids", "1,2,3", "--max-tokens",
                           "5", "--temperature", "0"], capture_output=True, text=True, timeout=600)
    assert chat.returncode == 0, chat.stderr[-2000:]
