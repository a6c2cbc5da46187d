"""Zudisun on the GPU against the plain implementation (``tests/plain_zudisun.py``) and the kernels' plain
twins: each new kernel alone, each mixer alone inside the engine, then whole models of several shapes
under every way of cutting requests into steps, with small pools so that pages and slots change hands,
in float32 (strict) and bfloat16."""

from __future__ import annotations

import copy
from typing import Dict, List

import pytest
import torch

import traces
from helpers import assert_close, make_runner, run_trace, save_model_folder
from plain_zudisun import (NO_CACHE, ODD, ONLY_SCAN, ONLY_SIGMOID, PAIR, plain_bucket, plain_zudisun_forward,
                           plain_zudisun_greedy, plain_zudisun_weights)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CONFIGS = {"pair": PAIR, "only_sigmoid": ONLY_SIGMOID, "only_scan": ONLY_SCAN, "odd": ODD, "no_cache": NO_CACHE}


def _tokens(config, lengths: Dict[str, int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {r: torch.randint(0, config["vocab"], (n,), generator=g).tolist() for r, n in lengths.items()}


def _close(got, want, dtype, what=""):
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), msg=lambda m: f"{what}: {m}", **tol)


def _routed(config) -> bool:
    return any((l.get("mlp") or {}).get("kind") == "moe" for l in config["layers"])


def _close_to_plain(got, want, noise, dtype, what, routed):
    """The engine against the plain run ``want``, with the plain run at the engine's precision (``noise``) as the
    yardstick: the worst error of that run over all the requests of the model is what rounding does there.
    float32 (``want``: the float64 run): three times that; bfloat16 (``want``: the float32 run): twice that, of
    which nine tenths may be used.  bfloat16 with routed experts: a routing decision that lies within rounding of
    a tie may fall the other way than in the plain bfloat16 run, and the positions that read that token then
    differ by more than rounding (a recurrent layer behind it carries the difference on for some tokens): nine in
    ten positions keep to the tolerance, and none is off by more than a routing decision can explain."""
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


def _i32(values) -> torch.Tensor:
    return torch.tensor(list(values), dtype=torch.int32)


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D", [(5, 40), (3, 200), (70, 1000)])
def test_stream_rows_with_an_output_bias_and_the_gated_activations(dtype, T, D):
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(T + D)
    h, delta = torch.randn(T, D, generator=g), torch.randn(T, D, generator=g).to(dtype)
    wp, bias = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype), torch.randn(D, generator=g)
    for with_delta in (True, False):
        hc, hg = h.clone(), h.clone().to(DEV)
        xc, xg = torch.empty(T, D, dtype=dtype), torch.empty(T, D, dtype=dtype, device=DEV)
        if with_delta:
            twins.post_add_rmsnorm(hc, delta, wp, 1e-5, None, 0.0, xc, delta_bias=bias)
            ops.post_add_rmsnorm(hg, delta.to(DEV), wp.to(DEV), 1e-5, None, 0.0, xg, delta_bias=bias.to(DEV))
        else:
            twins.post_add_rmsnorm(hc, None, None, 0.0, None, 0.0, xc)
            ops.post_add_rmsnorm(hg, None, None, 0.0, None, 0.0, xg)
        torch.testing.assert_close(hg.cpu(), hc, rtol=1e-5, atol=1e-5)
        _close(xg, xc, dtype, "the stream's rows")
    F = 8 * ((D + 15) // 16)
    gu, b = torch.randn(T, 2 * F, generator=g), torch.randn(2 * F, generator=g)
    for act in ("relu", "silu", "gelu_tanh"):
        for bb in (b, None):
            got = ops.gated_mul(gu.to(DEV), None if bb is None else bb.to(DEV), act, dtype)
            _close(got, twins.gated_mul(gu, bb, act, dtype), dtype, f"gated_mul {act}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,top,groups,keep", [(50, 6, 2, 3, 2), (200, 8, 4, 4, 3), (7, 8, 2, 8, 3), (30, 5, 5, 1, 1),
                                                  (90, 64, 6, 8, 4), (3, 4, 1, 1, 1), (40, 160, 8, 80, 5)])
def test_grouped_sigmoid_router_kernel(dtype, T, E, top, groups, keep):
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(E * 10 + top)
    D = 72
    x, router = torch.randn(T, D, generator=g).to(dtype), torch.randn(E, D, generator=g) / 4
    corr = torch.randn(E, generator=g) - 0.8
    want_c, want_w = twins.moe_route(x, router, None, top, True, corr, groups, keep, 1.5)
    got_c, got_w = ops.moe_route(x.to(DEV), router.to(DEV), None, top, True, corr.to(DEV), groups, keep, 1.5)
    assert torch.equal(got_c.cpu(), want_c), "the chosen experts, in the order of their choice scores"
    torch.testing.assert_close(got_w.cpu(), want_w, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,N,R,K,lens", [(10, 4, 3, 3, [5, 1, 8]), (70, 1, 1, 1, [4, 2]), (36, 37, 2, 9, [2, 1, 1, 30]),
                                          (256, 24, 10, 4, [130, 1, 1, 17]), (24, 300, 8, 2, [9, 3]), (8, 600, 8, 16, [20]),
                                          (48, 16, 4, 4, [300, 1, 70, 200]), (20, 5, 2, 3, [192])])
def test_convolution_and_scan_kernels_carry_their_state(dtype, C, N, R, K, lens):
    """Two steps of every sequence, through slots in another order: the kernels against their twins, the state
    and the convolution's tail after each step too."""
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(C + K)
    B = len(lens)
    taps, cb = torch.randn(C, K, generator=g) / K ** 0.5, torch.randn(C, generator=g)
    A, D, db = -torch.rand(C, N, generator=g) - 0.05, torch.randn(C, generator=g), torch.randn(C, generator=g) - 1.0
    state = torch.zeros(B + 1, C, N + K - 1)
    state[B] = 7.0
    state_g = state.clone().to(DEV)
    slots = _i32(reversed(range(B)))
    q_start = _i32([0] + torch.tensor(lens).cumsum(0).tolist())
    seq_of_token = torch.cat([torch.full((n,), b, dtype=torch.int32) for b, n in enumerate(lens)])
    T = sum(lens)
    for step in range(2):
        rows = torch.randn(T, 2 * C + 3, generator=g).to(dtype)  # [x | z | a few more columns]
        dt = torch.randn(T, C, generator=g)
        bc = (torch.randn(T, R + 2 * N, generator=g) / N ** 0.5).to(dtype)
        u, out = torch.empty(T, C, dtype=dtype), torch.empty(T, C, dtype=dtype)
        twins.causal_conv(rows, taps, cb, state, N, slots, seq_of_token, q_start, u, activation="silu")
        twins.selective_scan(u, dt, db, A, bc, R, R + N, D, rows[:, C:], rows, K, state, slots, q_start, B, out)
        rows_g, ug, og = rows.to(DEV), torch.empty(T, C, dtype=dtype, device=DEV), torch.empty(T, C, dtype=dtype, device=DEV)
        ops.causal_conv(rows_g, taps.to(DEV), cb.to(DEV), state_g, N, slots.to(DEV), seq_of_token.to(DEV), q_start.to(DEV), ug,
                        activation="silu")
        _close(ug, u, dtype, f"convolution, step {step}")
        # the scan from the twin's convolution, so that its own error alone is measured
        ops.selective_scan(u.to(DEV), dt.to(DEV), db.to(DEV), A.to(DEV), bc.to(DEV), R, R + N, D.to(DEV), rows_g[:, C:], rows_g, K,
                           state_g, slots.to(DEV), q_start.to(DEV), B, og, q_start_host=q_start.numpy())  # (long runs in chunks)
        _close(og, out, dtype, f"scan, step {step}")
        tol = 2e-5 if dtype == torch.float32 else 2e-3
        torch.testing.assert_close(state_g.cpu(), state, rtol=tol, atol=tol)
    assert float((state_g[B] - 7.0).abs().max()) == 0.0, "a slot that no sequence of the step holds stays"


def _paged(T, n_kv, hc, P, dtype, seed):
    """Pages filled with NaN, one sequence's table over them in a shuffled order, the slots of positions 0..T-1."""
    n_pages = -(-T // P) + 2
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed))[: -(-T // P)].tolist()
    kp = torch.full((n_pages, n_kv, P, hc), float("nan"), dtype=dtype)
    vp = torch.full((n_pages, n_kv, hc, P), float("nan"), dtype=dtype)
    table = torch.full((2, n_pages), -1, dtype=torch.int32)
    table[1, : len(order)] = _i32(order)
    slots = _i32(order[t // P] * P + t % P for t in range(T))
    return kp, vp, table, slots


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,e,hc,P,rows,far,every,T", [(4, 2, 6, 4, 8, 8, 6, 9.0, 3, 29), (8, 4, 80, 48, 80, 64, 24, 150.0, 100, 700),
                                                            (3, 3, 8, 10, 16, 16, 8, 40.0, 1, 150), (34, 2, 8, 8, 16, 16, 64, 33.0, 7, 90),
                                                            (5, 1, 20, 48, 48, 32, 9, 1000.0, 1000, 300),
                                                            (16, 4, 64, 64, 64, 64, 16, 600.0, 50, 1100), (12, 3, 32, 16, 32, 32, 10, 64.0, 9, 130),
                                                            (12, 4, 16, 16, 16, 32, 12, 90.0, 4, 200), (16, 16, 32, 32, 32, 64, 8, 20.0, 11, 150),
                                                            (3, 3, 8, 10, 16, 32, 8, 40.0, 1, 100), (1, 1, 24, 8, 32, 96, 6, 7.0, 2, 250)])
def test_prepare_and_sigmoid_attention_kernels(dtype, H, G, d, e, hc, P, rows, far, every, T):
    """Unit norms per head, the query's temperature, blended values, pages; then the attention over the pages for
    a whole prompt, for its last tokens alone with the keys cut over workgroups, and both with the same bits."""
    from fastgen_amd.kernels import ops, twins
    from fastgen_amd.parts.position import distance_table

    g = torch.Generator().manual_seed(H * 7 + d)
    src = torch.randn(T, H * d + G * d + G * e + H, generator=g)
    v_first = torch.randn(T, G * e + 3, generator=g)
    rel, talk = torch.randn(rows, H, generator=g), torch.eye(H) + 0.3 * torch.randn(H, H, generator=g) / H ** 0.5
    pb = torch.randn(H, generator=g) - 3.0
    spread = distance_table(rel, far).contiguous()
    kp, vp, table, slots = _paged(T, G, hc, P, dtype, T)
    pos, seq = torch.arange(T, dtype=torch.int32), torch.ones(T, dtype=torch.int32)
    common = dict(n_q=H, q_col=0, q_width=d, q_norm_dims=d, q_out_width=d, n_kv=G, k_col=H * d, k_width=d, k_norm_dims=d,
                  v_col=H * d + G * d, v_width=e, norm_plain=True, q_temp_coef=0.75, q_temp_every=every, v_blend=0.3)
    q = torch.empty(T, H * d, dtype=dtype)
    twins.heads_prepare(src, None, 1e-5, q_out=q, slots=slots, k_pages=kp, v_pages=vp, positions=pos, v_first=v_first, **common)
    qg, kg, vg = torch.empty(T, H * d, dtype=dtype, device=DEV), kp.to(DEV), vp.to(DEV)
    ops.heads_prepare(src.to(DEV), None, 1e-5, q_out=qg, slots=slots.to(DEV), k_pages=kg, v_pages=vg, positions=pos.to(DEV),
                      v_first=v_first.to(DEV), **common)
    _close(qg, q, dtype, "queries")
    written = ~torch.isnan(kp.float())
    assert torch.equal(~torch.isnan(kg.float().cpu()), written), "keys are written at the tokens' slots alone"
    _close(kg.cpu()[written], kp[written], dtype, "keys")
    written = ~torch.isnan(vp.float())
    _close(vg.cpu()[written], vp[written], dtype, "values")
    gate = src[:, H * d + G * d + G * e :].contiguous()
    out = torch.empty(T, H * e, dtype=dtype)
    twins.sigmoid_attention(q, d, out, e, kp, vp, table, seq, pos, H, 0.4, spread, talk, pb, gate)
    kg, vg = kp.to(DEV), vp.to(DEV)  # the twin's pages: the attention's own error alone
    args = (kg, vg, table.to(DEV))
    rest = (H, 0.4, spread.to(DEV), talk.to(DEV), pb.to(DEV))
    og = torch.empty(T, H * e, dtype=dtype, device=DEV)
    ops.sigmoid_attention(q.to(DEV), d, og, e, *args, seq.to(DEV), pos.to(DEV), *rest, gate.to(DEV))
    tol = dict(rtol=3e-5, atol=3e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(og.float().cpu(), out.float(), **tol)
    last = slice(T - 3, T)
    cut = torch.empty(3, H * e, dtype=dtype, device=DEV)
    ops.sigmoid_attention(q[last].to(DEV), d, cut, e, *args, seq[last].to(DEV), pos[last].to(DEV), *rest,
                          gate[last].contiguous().to(DEV), split_for=T)
    assert torch.equal(cut, og[last]), "keys cut over workgroups: the same bits"
    if dtype == torch.bfloat16 and P % 32 == 0 and H <= ops.SIGMOID_TILE_HEADS:
        # prompt portions on the matrix cores: the whole prompt, and its last 40 tokens behind the cached rest
        mixed = ops.sigmoid_attention_mixed(0.4, H, spread.to(DEV), talk.to(DEV), pb.to(DEV), DEV)
        items = ops.upload(ops.sigmoid_attention_items([0, T], [0, 0, T], [0, 0]), torch.int32, DEV)
        assert int(items[:, 2].sum()) == T and int(items[:, 2].max()) <= 16
        tiles = torch.empty(T, H * e, dtype=dtype, device=DEV)
        ops.sigmoid_attention(q.to(DEV), d, tiles, e, *args, seq.to(DEV), pos.to(DEV), *rest, gate.to(DEV), split_for=T,
                              items=items, mixed=mixed)
        torch.testing.assert_close(tiles.float().cpu(), out.float(), **tol)
        part = slice(T - 40, T)
        items = ops.upload(ops.sigmoid_attention_items([0, 40], [0, 0, 40], [0, T - 40]), torch.int32, DEV)
        tiles = torch.empty(40, H * e, dtype=dtype, device=DEV)
        ops.sigmoid_attention(q[part].to(DEV), d, tiles, e, *args, seq[part].to(DEV), pos[part].to(DEV), *rest,
                              gate[part].contiguous().to(DEV), split_for=T, items=items, mixed=mixed)
        torch.testing.assert_close(tiles.float().cpu(), out[part].float(), **tol)
        # single tokens of three sequences (here: three positions of one), the keys in many small chunks
        singles = ops.upload([[1, 0, 1, T - 3], [1, 1, 1, T - 2], [1, 2, 1, T - 1]], torch.int32, DEV)
        ops.sigmoid_attention(q[last].to(DEV), d, cut, e, *args, seq[last].to(DEV), pos[last].to(DEV), *rest,
                              gate[last].contiguous().to(DEV), split_for=T + 200, items=singles, mixed=mixed)
        torch.testing.assert_close(cut.float().cpu(), out[last].float(), **tol)
        plain = ops.sigmoid_attention_mixed(0.4, H, None, None, pb.to(DEV), DEV)
        twins.sigmoid_attention(q[part], d, out[part], e, kp, vp, table, seq[part], pos[part], H, 0.4, None, None, pb, None)
        ops.sigmoid_attention(q[part].to(DEV), d, tiles, e, *args, seq[part].to(DEV), pos[part].to(DEV), H, 0.4, None, None,
                              pb.to(DEV), None, split_for=T, items=items, mixed=plain)
        torch.testing.assert_close(tiles.float().cpu(), out[part].float(), **tol)
    # without the optional parts
    twins.sigmoid_attention(q, d, out, e, kp, vp, table, seq, pos, H, 0.4, None, None, pb, None)
    ops.sigmoid_attention(q.to(DEV), d, og, e, *args, seq.to(DEV), pos.to(DEV), H, 0.4, None, None, pb.to(DEV), None)
    torch.testing.assert_close(og.float().cpu(), out.float(), **tol)


# ----------------------------------------------------------------- whole models
LENGTHS = {"a": 150, "b": 37, "c": 2, "d": 1, "e": 70, "f": 19}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        weights = plain_zudisun_weights(config, seed=len(name))
        folder = save_model_folder(tmp_path_factory.mktemp(name), config, weights)
        toks = _tokens(config, LENGTHS, seed=7)
        out[name] = (config, weights, folder, toks, {r: plain_zudisun_forward(config, weights, t) for r, t in toks.items()})
    return out


@pytest.fixture(scope="module")
def exact(cases):
    """The float64 runs of the same requests: what float32 results are measured against where sums are long."""
    return {name: {r: plain_zudisun_forward(c[0], c[1], t, torch.float64) for r, t in c[3].items()} for name, c in cases.items()}


def _all_traces(lengths):
    return {"whole": traces.whole(lengths), "tail": traces.tail(lengths, 60), "chunks": traces.chunks(lengths),
            "pairs": traces.chunks(lengths, sizes=(2, 3, 2, 5)),
            "mixed": traces.mixed(lengths, seed=3), "mixed2": traces.mixed(lengths, max_live=3, seed=11, budget=23)}


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_float32_every_cut_batch_and_reuse(cases, exact, name):
    """Whole prompts, prompts then single tokens, portions down to two tokens and one, mixed batches of unequal
    requests: the same logits as the plain run whatever the cut.  Pages of 16 tokens and a pool that holds the
    live requests only: pages and state slots are used again."""
    config, weights, folder, toks, want = cases[name]
    runner = make_runner(folder, torch.float32, page_size=16, max_tokens=304, max_requests=4)
    first = None
    for kind, tr in _all_traces(LENGTHS).items():
        got = run_trace(runner, tr, toks)
        _close_to_plain(got, exact[name], want, torch.float32, f"zudisun {name} {kind}", _routed(config))
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
    noise = {r: plain_zudisun_forward(config, weights, t, torch.bfloat16) for r, t in toks.items()}
    for page, pool in ((16, 304), (64, 768)):  # (pages of 64: prompt portions of the attention run on the matrix cores)
        runner = make_runner(folder, torch.bfloat16, page_size=page, max_tokens=pool, max_requests=4)
        for kind, tr in _all_traces(LENGTHS).items():
            _close_to_plain(run_trace(runner, tr, toks), want, noise, torch.bfloat16, f"zudisun {name} {kind} bfloat16, pages of {page}",
                            _routed(config))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_streams_after_every_layer(cases, dtype):
    """The residual stream after each layer, read from the engine by stopping the run order there."""
    import dataclasses

    from fastgen_amd.engine import Model, ModelRunner, StepEntry
    from fastgen_amd.kernels import ops
    from fastgen_amd.weights.source import SafetensorsSource

    config, weights, folder, toks, _ = cases["pair"]
    streams: list = []
    plain_zudisun_forward(config, weights, toks["b"], dtype, layers_out=streams)
    full = Model.from_folder(folder, dtype, DEV)
    for n_runs in range(1, len(full.layout.order) + 1):
        layout = dataclasses.replace(full.layout, order=full.layout.order[:n_runs])
        model = Model(layout, dtype, DEV, args=full.args, architecture=full.architecture)
        model.load(SafetensorsSource(folder))
        seen = {}
        norm = model.parts.final_norm
        keep = norm.forward
        norm.forward = lambda h, pending, dt, rows=None: (seen.update(h=h.clone(), pending=pending), keep(h, pending, dt, rows))[1]
        runner = ModelRunner(model, page_size=16, max_tokens=64, max_requests=1)
        runner.step([StepEntry("b", toks["b"], [0])])
        h, pending = seen["h"], seen["pending"]
        ops.post_add_rmsnorm(h, pending.rows, pending.weight, pending.eps, None, 0.0, None, delta_bias=pending.bias)
        want = streams[n_runs - 1]
        tol = 2e-5 if dtype == torch.float32 else 4e-2
        off = ((h.cpu() - want).abs().amax(-1) > tol * float(want.abs().max())).nonzero().flatten().tolist()
        # bfloat16: a token whose routing decision is a close call may get another expert than in the plain run
        assert len(off) <= (0 if dtype == torch.float32 else 0.1 * len(toks["b"])), f"after {n_runs} layers: rows {off}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["pair", "odd"])
def test_long_decoding_across_pages(cases, dtype, name):
    """A short prompt, then 290 tokens one by one over many pages: the distance table's last row, every step of the
    temperature, the recurrence over 290 steps (bfloat16: recorded steps)."""
    config, weights, folder, _, _ = cases[name]
    toks = _tokens(config, {"z": 300}, seed=5)
    want = {"z": plain_zudisun_forward(config, weights, toks["z"])}
    runner = make_runner(folder, dtype, page_size=16, max_tokens=304, max_requests=2)
    got = run_trace(runner, traces.tail({"z": 300}, 290), toks)
    if dtype == torch.float32:
        _close_to_plain(got, {"z": plain_zudisun_forward(config, weights, toks["z"], torch.float64)}, want, dtype,
                        f"zudisun {name} long decoding", True)
    else:
        _close_to_plain(got, want, {"z": plain_zudisun_forward(config, weights, toks["z"], torch.bfloat16)}, dtype,
                        f"zudisun {name} long decoding bfloat16", True)


@pytest.mark.parametrize("name", ["pair", "no_cache"])
def test_long_prompts_beside_short_ones(cases, name):
    """Prompts of several hundred tokens in one step, together in one batch, in two steps and in small portions."""
    config, weights, folder, _, _ = cases[name]
    lengths = {"p": 700, "q": 260, "r": 3}
    toks = _tokens(config, lengths, seed=13)
    want = {r: plain_zudisun_forward(config, weights, t) for r, t in toks.items()}
    exact = {r: plain_zudisun_forward(config, weights, t, torch.float64) for r, t in toks.items()}
    noise = {r: plain_zudisun_forward(config, weights, t, torch.bfloat16) for r, t in toks.items()}
    together = [([("p", 0, 700), ("q", 0, 260), ("r", 0, 3)], ["p", "q", "r"])]
    for dtype, page in ((torch.float32, 16), (torch.bfloat16, 16), (torch.bfloat16, 64)):
        runner = make_runner(folder, dtype, page_size=page, max_tokens=1152, max_requests=3)
        for kind, tr in (("whole", traces.whole(lengths)), ("together", together),
                         ("halves", traces.chunks(lengths, sizes=(390, 310))), ("portions", traces.chunks(lengths))):
            got = run_trace(runner, tr, toks)
            if dtype == torch.float32:
                _close_to_plain(got, exact, want, dtype, f"zudisun {name} long {kind}", True)
            else:
                _close_to_plain(got, want, noise, dtype, f"zudisun {name} long {kind} bfloat16", True)


def test_the_scan_remembers_a_far_token(tmp_path):
    """With decays close to one the state carries tokens for hundreds of steps: the logits at the end follow the
    first 40 tokens, 300 positions back, in a prompt, in portions and decoded alone, and through a slot that
    another request held before; losing the state (or starting from another request's) would change them by far
    more than the tolerance."""
    config = copy.deepcopy(ONLY_SCAN)
    w = plain_zudisun_weights(config, 3)
    w["l0.mix.A_log"][:] = -7.0  # A = -0.0009: a decay of 0.9999 a step and more
    w["l0.mix.dt.b"][:] = -1.0
    n = 330
    toks = _tokens(config, {"other": 50, "s": n}, seed=2)
    want = {r: plain_zudisun_forward(config, w, t) for r, t in toks.items()}
    without = list(toks["s"])
    for i in range(40):
        without[i] = (without[i] + 1) % config["vocab"]
    gap = float((plain_zudisun_forward(config, w, without)[-1] - want["s"][-1]).abs().max())
    assert gap > 0.02 * float(want["s"].abs().max()), "the test's weights do not make the far tokens count"
    folder = save_model_folder(tmp_path / "m", config, w)
    lengths = {"other": 50, "s": n}
    for dtype in (torch.float32, torch.bfloat16):
        runner = make_runner(folder, dtype, page_size=16, max_tokens=64, max_requests=1)  # one slot: it is used again
        for tr in (traces.whole(lengths), traces.tail(lengths, 25), traces.chunks(lengths), traces.chunks(lengths, sizes=(2, 3, 2))):
            got = run_trace(runner, tr, toks)
            if dtype == torch.float32:
                assert_close(got, want, dtype, None, "far token")
            else:
                assert float((got["s"][-1] - want["s"][-1]).abs().max()) < 0.25 * gap


def test_keys_at_the_edges_of_the_distance_table(tmp_path):
    """One layer of attention whose scores are the distance bias alone, with one row of the table far above the
    others: a query adds up exactly the values of the keys whose distance falls into that row, so a distance
    that is one off, at a step of the table, at a page's border, for the first keys of a sequence or for keys
    hundreds of tokens back, changes the logits by far more than the tolerance.  Whole prompts, portions down to
    two tokens, decoding alone."""
    n = 230
    for row, far in ((3, 50.0), (9, 50.0), (12, 50.0), (15, 50.0), (15, 200.0)):
        config = copy.deepcopy(ONLY_SIGMOID)
        config["layers"][0]["mixer"]["bias_max"] = far
        w = plain_zudisun_weights(config, row)
        w["l0.mix.q"][:] = 0.0
        w["l0.mix.talk"] = torch.eye(2)
        w["l0.mix.pb"][:] = -6.0
        w["l0.mix.rel"][:] = -14.0
        w["l0.mix.rel"][row] = 14.0
        w["l0.mix.v"] *= 0.25 if row == 15 else 1.0  # the last row holds every far key
        toks = _tokens(config, {"s": n}, seed=row)
        want = {"s": plain_zudisun_forward(config, w, toks["s"])}
        lo = min(d for d in range(n) if plain_bucket(d, 16, far) == row)
        # the key at the row's first distance counts: without it the logits move
        other = copy.deepcopy(config)
        other["layers"][0]["mixer"]["bias_max"] = far * 1.3
        moved = (plain_zudisun_forward(other, w, toks["s"]) - want["s"]).abs().amax(-1)
        if row >= 9:
            assert float(moved[lo + 5 :].min()) > 0.02 * float(want["s"].abs().max()), "the table's steps do not decide"
        folder = save_model_folder(tmp_path / f"r{row}_{int(far)}", config, w)
        for dtype, page in ((torch.float32, 16), (torch.bfloat16, 16), (torch.bfloat16, 64)):
            runner = make_runner(folder, dtype, page_size=page, max_tokens=256, max_requests=1)
            noise = {"s": plain_zudisun_forward(config, w, toks["s"], torch.bfloat16)} if dtype == torch.bfloat16 else None
            for tr in (traces.whole({"s": n}), traces.tail({"s": n}, 170), traces.chunks({"s": n}),
                       traces.chunks({"s": n}, sizes=(2, 3, 2, 5))):
                assert_close(run_trace(runner, tr, {"s": toks["s"]}), want, dtype, noise, f"row {row} far {far}")


def test_greedy_generation_through_the_engine(cases):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    config, weights, folder, toks, _ = cases["pair"]
    prompts = [toks["b"], toks["f"], toks["c"], toks["e"][:40], toks["d"]]
    want = [plain_zudisun_greedy(config, weights, p, 9) for p in prompts]
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
