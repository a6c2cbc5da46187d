"""Zudisun without a GPU: its configuration reader and layout, the plain implementation's own
mechanisms against hand-made cases, and the kernels' plain twins against the plain mechanisms."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from fastgen_amd.config import ConfigError, get_architecture
from fastgen_amd.engine.model import build_parts
from fastgen_amd.kernels import twins
from fastgen_amd.parts.position import distance_table, log_bucket
from plain_zudisun import (NO_CACHE, ODD, ONLY_SCAN, ONLY_SIGMOID, PAIR, plain_bucket, plain_causal_conv, plain_gated_ff,
                           plain_query_temperature, plain_rms, plain_route, plain_selective_scan, plain_sigmoid_attention,
                           plain_silu, plain_zudisun_forward, plain_zudisun_shapes, plain_zudisun_weights)

CONFIGS = {"pair": PAIR, "only_sigmoid": ONLY_SIGMOID, "only_scan": ONLY_SCAN, "odd": ODD, "no_cache": NO_CACHE}


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_layout_names_every_tensor_and_the_configuration_round_trips(name):
    config = CONFIGS[name]
    arch = get_architecture(config)
    assert arch.name == "Zudisun"
    args = arch.parse(config)
    assert arch.parse(arch.to_hf_config(args)) == args
    specs = {s.name: tuple(s.shape) for s in build_parts(arch.layout(args)).tensor_specs()}
    assert specs == plain_zudisun_shapes(config)


def test_sizes_and_tensors_that_only_the_checkpoint_gives():
    config = copy.deepcopy(ONLY_SIGMOID)
    del config["layers"][0]["mixer"]["bias_rows"]
    arch = get_architecture(config)
    assert arch.parse(config).layers[0].mixer.bias_rows == 32
    shapes = {"l0.mix.rel": (20, 2), "l0.mix.vmix": ()}
    args = arch.parse(config, lambda name: shapes.get(name))  # the table's rows; a mixing number that is not used
    assert args.layers[0].mixer.bias_rows == 20 and not args.layers[0].mixer.v_mix
    specs = {s.name: tuple(s.shape) for s in build_parts(arch.layout(args)).tensor_specs()}
    assert specs["l0.mix.rel"] == (20, 2) and specs["l0.mix.vmix"] == ()


def test_what_the_mixers_ask_of_the_cache():
    arch = get_architecture(PAIR)
    parts = build_parts(arch.layout(arch.parse(PAIR)))
    scan, sig = parts.mixers[0], parts.mixers[1]
    assert scan.paged_need() is None and scan.state_need().shape == (96, 8 + 4 - 1)
    assert scan.state_need().dtype == torch.float32
    assert sig.state_need() is None and sig.paged_need().n_kv_heads == 2 and sig.paged_need().head_dim == 32
    one_tap = build_parts(arch.layout(arch.parse(ODD))).mixers[1]
    assert one_tap.state_need().shape == (70, 1)  # a state of one value and no tail
    only = build_parts(arch.layout(arch.parse(NO_CACHE)))
    assert all(m.paged_need() is None for m in only.mixers)


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].update(type="mamba2"), "not supported"),
    (lambda c: c["layers"][1]["mixer"].update(heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].update(bias_max=5), "bias_max"),
    (lambda c: c["layers"][1]["mixer"]["q_temp"].update(every=0), "q_temp.every"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=8), "agree in kv_heads and vdim"),
    (lambda c: c["layers"][0]["mixer"].update(conv=0), "conv"),
    (lambda c: c["layers"][0]["mixer"].pop("state"), "state"),
    (lambda c: c["layers"][0]["mlp"].update(kind="switch"), "not supported"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "top"),
    (lambda c: c["norm"].pop("eps"), "norm.eps"),
])
def test_configuration_errors_name_what_is_wrong(change, match):
    config = copy.deepcopy(PAIR)
    change(config)
    with pytest.raises(ConfigError, match=match):
        get_architecture(config).parse(config)


# ------------------------------------------------- the plain mechanisms on hand-made cases
def test_plain_buckets_and_the_spread_table():
    # 12 rows, far 30: one row a distance below 6, the last row from 30 on, steps in between that never go back
    rows = [plain_bucket(n, 12, 30.0) for n in range(40)]
    assert rows[:6] == list(range(6)) and rows[6] == 6 and rows[29] == 11 and set(rows[30:]) == {11}
    assert all(b >= a for a, b in zip(rows, rows[1:]))
    assert plain_bucket(12, 12, 30.0) == 6 + int(math.log(2.0) / math.log(5.0) * 6)
    # an odd number of rows: half is rounded down
    assert [plain_bucket(n, 7, 5.0) for n in range(7)] == [0, 1, 2, 3, 5, 6, 6]
    for n_rows, far in ((12, 30.0), (7, 5.0), (9, 1000.0), (64, 33.0), (7, 64.5), (32, 200.0)):
        table = torch.arange(n_rows, dtype=torch.float32)[:, None] * torch.tensor([1.0, -2.0])
        spread = distance_table(table, far)
        assert spread.shape[0] == math.ceil(far) + 1
        for n in range(spread.shape[0] + 5):
            want = plain_bucket(n, n_rows, far)
            assert log_bucket(n, n_rows, far) == want
            assert float(spread[min(n, spread.shape[0] - 1), 0]) == want
    with pytest.raises(ValueError):
        distance_table(torch.zeros(8, 2), 4.0)


def test_plain_temperature_conv_and_scan():
    t = plain_query_temperature(torch.tensor([0, 2, 3, 6, 7, 11]), 0.5, 4)
    want = [1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(3), 1 + 0.5 * math.log(4)]
    torch.testing.assert_close(t, torch.tensor(want, dtype=t.dtype))
    # the last tap meets the token itself; zeros before the start
    u = torch.tensor([[1.0], [2.0], [4.0]])
    y = plain_causal_conv(u, torch.tensor([[100.0, 10.0, 1.0]]), torch.tensor([0.5]))
    torch.testing.assert_close(y, torch.tensor([[1.5], [12.5], [124.5]]))
    # one channel, one state: S <- exp(d a) S + d u b, y = S c + D u
    d, a = torch.tensor([[0.5], [0.25]]), torch.tensor([[-2.0]])
    y = plain_selective_scan(torch.tensor([[3.0], [-1.0]]), d, a, torch.tensor([[2.0], [1.0]]), torch.tensor([[1.0], [4.0]]),
                             torch.tensor([10.0]))
    s0 = 0.5 * 3.0 * 2.0
    s1 = math.exp(-0.5) * s0 + 0.25 * -1.0 * 1.0
    torch.testing.assert_close(y, torch.tensor([[s0 + 30.0], [4 * s1 - 10.0]]))


def test_plain_sigmoid_attention_is_its_definition():
    g = torch.Generator().manual_seed(1)
    T, H, G, d, e, rows, far = 9, 4, 2, 6, 3, 6, 7.0
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, G, d, generator=g), torch.randn(T, G, e, generator=g)
    rel, talk, pb = torch.randn(rows, H, generator=g), torch.randn(H, H, generator=g), torch.randn(H, generator=g)
    got = plain_sigmoid_attention(q, k, v, 0.3, rel, far, talk, pb)
    for i in (0, 3, 8):
        want = torch.zeros(H, e)
        for j in range(i + 1):
            s = torch.stack([(q[i, h] @ k[j, h // 2]) * 0.3 + rel[plain_bucket(i - j, rows, far), h] for h in range(H)])
            w = torch.sigmoid(talk @ s + pb)
            want += w[:, None] * v[j].repeat_interleave(2, dim=0)
        torch.testing.assert_close(got[i], want, rtol=1e-5, atol=1e-5)
    # the weights are not normalised: with a huge head bias every key counts once
    got = plain_sigmoid_attention(q, k, v, 0.3, rel, far, torch.eye(H), torch.full((H,), 40.0))
    torch.testing.assert_close(got[:, 0], v[:, 0].cumsum(0), rtol=1e-5, atol=1e-5)


def test_plain_route_groups_correction_and_weights():
    # 6 experts in 3 groups; logits through an identity router
    router, none = torch.eye(6), torch.zeros(6)
    x = torch.tensor([[2.0, 1.9, 3.0, -5.0, 1.0, 1.2]])
    # group sums of the two largest scores: (0,1) .88+.87, (2,3) .95+.007, (4,5) .73+.77: the group of expert 2 loses
    chosen, w = plain_route(x, router, none, 2, 3, 2, 2.0)
    assert sorted(chosen[0].tolist()) == [0, 1]
    s = torch.sigmoid(x[0, :2])
    torch.testing.assert_close(w[0].sum(), torch.tensor(2.0))
    torch.testing.assert_close(w[0], 2.0 * s[chosen[0]] / s.sum())
    # all groups stay: the largest scores win wherever they are
    assert sorted(plain_route(x, router, none, 2, 3, 3, 1.0)[0][0].tolist()) == [0, 2]
    # the correction moves the choice and not the weights
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 1.0])
    chosen, w = plain_route(x, router, corr, 2, 1, 1, 1.0)
    assert sorted(chosen[0].tolist()) == [2, 5]
    s = torch.sigmoid(x[0, [2, 5]])
    torch.testing.assert_close(w[0].sort().values, (s / s.sum()).sort().values)
    # negative choice scores: an expert of a group that lost is not chosen although its score is larger
    corr = torch.tensor([-3.0, -3.0, -2.0, -2.0, -9.0, -9.0])
    assert sorted(plain_route(x, router, corr, 3, 3, 2, 1.0)[0][0].tolist())[-1] <= 3


def test_every_mechanism_moves_the_logits():
    """The random weights of these tests are large enough that leaving a mechanism out shows."""
    toks = torch.randint(0, PAIR["vocab"], (60,), generator=torch.Generator().manual_seed(4)).tolist()
    w = plain_zudisun_weights(PAIR, 1)
    base = plain_zudisun_forward(PAIR, w, toks)
    scale = float(base.abs().max())

    def moved(change_w=None, change_c=None):
        w2, c2 = {k: v.clone() for k, v in w.items()}, copy.deepcopy(PAIR)
        if change_w:
            change_w(w2)
        if change_c:
            change_c(c2)
        return float((plain_zudisun_forward(c2, w2, toks) - base).abs().max()) / scale

    assert moved(lambda w2: w2["l1.mix.rel"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l1.mix.talk"].copy_(torch.eye(4))) > 1e-3
    assert moved(lambda w2: w2["l1.mix.pb"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l1.mix.g"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l2.mix.vmix"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l4.mix.vmix"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l1.mix.vmix"].add_(1.0)) == 0.0  # the first mixing layer's number is not used
    assert moved(lambda w2: w2["l0.mix.conv.b"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l0.mix.conv"][:, 0].zero_()) > 1e-3
    assert moved(lambda w2: w2["l0.mix.D"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l3.mix.dt.b"].add_(1.0)) > 1e-3
    assert moved(lambda w2: w2["l0.mlp.correction"].mul_(-4.0)) > 1e-3
    assert moved(lambda w2: w2["l0.mlp.shared.down"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l1.mlp.down.b"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l1.mlp.gate.b"].zero_()) > 1e-3
    assert moved(change_c=lambda c: c["layers"][1]["mixer"].update(bias_max=60)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][2]["mixer"]["q_temp"].update(every=6)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][2]["mixer"]["q_temp"].update(coef=0.0)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][1]["mixer"].update(scale=0.3)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=3)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][0]["mlp"]["router"].update(scale=1.0)) > 1e-3
    assert moved(change_c=lambda c: c["norm"].update(eps=1e-2)) > 1e-4


# ------------------------------------------------- the kernels' twins against the plain mechanisms
def test_twins_of_the_row_kernels():
    g = torch.Generator().manual_seed(5)
    T, D = 6, 40
    h, delta, bias = torch.randn(T, D, generator=g), torch.randn(T, D, generator=g), torch.randn(D, generator=g)
    wp = 1 + 0.1 * torch.randn(D, generator=g)
    # the stream's own rows, with what is pending (a sublayer's output plus its last bias, normed) added first
    hh, x = h.clone(), torch.empty(T, D)
    twins.post_add_rmsnorm(hh, delta, wp, 1e-5, None, 0.0, x, delta_bias=bias)
    torch.testing.assert_close(hh, h + plain_rms(delta + bias, wp, 1e-5))
    torch.testing.assert_close(x, hh)
    hh = h.clone()
    twins.post_add_rmsnorm(hh, None, None, 0.0, None, 0.0, x)
    torch.testing.assert_close(hh, h)
    torch.testing.assert_close(x, h)
    # gate and up interleaved in groups of 8, their biases in that order
    F = 24
    gate, up = torch.randn(T, F, generator=g), torch.randn(T, F, generator=g)
    bg, bu = torch.randn(F, generator=g), torch.randn(F, generator=g)
    gu = twins.interleave_gate_up(gate.T.contiguous(), up.T.contiguous()).T.contiguous()
    b = twins.interleave_gate_up(bg[:, None], bu[:, None])[:, 0]
    torch.testing.assert_close(twins.gated_mul(gu, b, "relu", torch.float32), torch.relu(gate + bg) * (up + bu))
    torch.testing.assert_close(twins.gated_mul(gu, None, "silu", torch.float32), plain_silu(gate) * up)
    w = {"p.gate": torch.randn(F, D, generator=g), "p.up": torch.randn(F, D, generator=g), "p.down": torch.randn(D, F, generator=g),
         "p.gate.b": bg, "p.up.b": bu, "p.down.b": bias}
    xin = torch.randn(T, D, generator=g)
    gu = torch.cat([xin @ w["p.gate"].T, xin @ w["p.up"].T], dim=1)
    gu = twins.interleave_gate_up((xin @ w["p.gate"].T).T.contiguous(), (xin @ w["p.up"].T).T.contiguous()).T.contiguous()
    got = twins.gated_mul(gu, b, "relu", torch.float32) @ w["p.down"].T + bias
    torch.testing.assert_close(got, plain_gated_ff(xin, w, "p", torch.float32, "relu", True), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("E,top,groups,keep,scale", [(6, 2, 3, 2, 2.0), (8, 4, 4, 3, 1.5), (8, 2, 8, 3, 1.0), (5, 5, 1, 1, 0.5),
                                                      (12, 3, 2, 1, 1.0), (4, 1, 1, 1, 1.0)])
def test_twin_of_the_grouped_sigmoid_router(E, top, groups, keep, scale):
    g = torch.Generator().manual_seed(E * 10 + top)
    T, D = 50, 24
    x, router = torch.randn(T, D, generator=g), torch.randn(E, D, generator=g)
    corr = torch.randn(E, generator=g) - 0.8  # choice scores of both signs
    want_c, want_w = plain_route(x, router, corr, top, groups, keep, scale)
    got_c, got_w = twins.moe_route(x, router, None, top, True, corr, groups, keep, scale)
    order_w, order_g = want_c.sort(dim=1), got_c.long().sort(dim=1)
    assert torch.equal(order_w.values, order_g.values)
    torch.testing.assert_close(got_w.gather(1, order_g.indices), want_w.gather(1, order_w.indices))


@pytest.mark.parametrize("C,N,R,K,lens", [(10, 4, 3, 3, [5, 1, 8]), (6, 1, 1, 1, [4, 2]), (7, 9, 2, 5, [2, 1, 1, 3])])
def test_twins_of_the_convolution_and_the_scan_carry_their_state(C, N, R, K, lens):
    """Two steps of every sequence through slots in another order: the same as the plain functions on the whole."""
    g = torch.Generator().manual_seed(C + K)
    B = len(lens)
    taps, cb = torch.randn(C, K, generator=g), torch.randn(C, generator=g)
    A, D, db = -torch.rand(C, N, generator=g) - 0.1, torch.randn(C, generator=g), torch.randn(C, generator=g)
    full = [dict(x=torch.randn(2 * n, C, generator=g), z=torch.randn(2 * n, C, generator=g), dt=torch.randn(2 * n, C, generator=g),
                 bc=torch.randn(2 * n, 1 + 2 * N, generator=g)) for n in lens]
    state = torch.zeros(B + 1, C, N + K - 1)
    state[B] = 7.0  # a slot that no sequence holds
    slots = torch.tensor(list(reversed(range(B))), dtype=torch.int32)
    q_start = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    seq_of_token = torch.cat([torch.full((n,), b, dtype=torch.int32) for b, n in enumerate(lens)])
    got = [[] for _ in lens]
    for half in range(2):
        cut = lambda key: torch.cat([f[key][half * n : (half + 1) * n] for f, n in zip(full, lens)])
        x, z, dt, bc = cut("x"), cut("z"), cut("dt"), cut("bc")
        u = torch.empty(x.shape)
        twins.causal_conv(x, taps, cb, state, N, slots, seq_of_token, q_start, u, activation="silu")
        out = torch.empty(x.shape)
        twins.selective_scan(u, dt, db, A, bc, 1, 1 + N, D, z, x, K, state, slots, q_start, B, out)
        for b in range(B):
            got[b].append(out[int(q_start[b]) : int(q_start[b + 1])])
    for b, f in enumerate(full):
        u = plain_silu(plain_causal_conv(f["x"], taps, cb))
        step = torch.nn.functional.softplus(f["dt"] + db)
        y = plain_selective_scan(u, step, A, f["bc"][:, 1 : 1 + N], f["bc"][:, 1 + N :], D) * plain_silu(f["z"])
        torch.testing.assert_close(torch.cat(got[b]), y, rtol=1e-5, atol=1e-5)
        if K > 1:
            padded = torch.cat([torch.zeros(K - 1, C), f["x"]])  # zeros before the start where the sequence is shorter
            torch.testing.assert_close(state[int(slots[b]), :, N:], padded[-(K - 1):].T)
    assert float((state[B] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("H,G,d,e,hc,P,rows,far,every", [(4, 2, 6, 4, 8, 8, 6, 9.0, 3), (3, 3, 8, 10, 16, 16, 8, 40.0, 1),
                                                          (5, 1, 4, 4, 8, 8, 5, 100.0, 1000)])
def test_twins_of_an_attention_layers_path(H, G, d, e, hc, P, rows, far, every):
    """Prepare (unit norms per head, the query's temperature, blended values, pages) and the attention over the
    pages with the spread table, mixed heads, head biases and gates: against the plain attention."""
    g = torch.Generator().manual_seed(H * 7 + d)
    T = 29
    src = torch.randn(T, H * d + G * d + G * e + H, generator=g)
    v_first = torch.randn(T, G * e + 3, generator=g)
    rel, talk, pb = torch.randn(rows, H, generator=g), torch.randn(H, H, generator=g), torch.randn(H, generator=g) - 1.0
    n_pages = 5
    kp, vp = torch.full((n_pages, G, P, hc), float("nan")), torch.full((n_pages, G, hc, P), float("nan"))
    table = torch.tensor([[4, 0, 2, 1]], dtype=torch.int32)
    slots = torch.tensor([int(table[0, t // P]) * P + t % P for t in range(T)], dtype=torch.int32)
    pos = torch.arange(T, dtype=torch.int32)
    q = torch.empty(T, H * d)
    twins.heads_prepare(src, None, 1e-5, n_q=H, q_col=0, q_width=d, q_norm_dims=d, q_out=q, q_out_width=d,
                        n_kv=G, k_col=H * d, k_width=d, k_norm_dims=d, v_col=H * d + G * d, v_width=e,
                        slots=slots, k_pages=kp, v_pages=vp, norm_plain=True, positions=pos, q_temp_coef=0.75,
                        q_temp_every=every, v_first=v_first, v_blend=0.3)
    out = torch.empty(T, H * e)
    gate = src[:, H * d + G * d + G * e :]
    twins.sigmoid_attention(q, d, out, e, kp, vp, table, torch.zeros(T, dtype=torch.int32), pos, H, 0.4,
                            distance_table(rel, far).contiguous(), talk, pb, gate)
    pq = plain_rms(src[:, : H * d].view(T, H, d), None, 1e-5)
    pq = pq * plain_query_temperature(pos, 0.75, every).float()[:, None, None]
    pk = plain_rms(src[:, H * d : H * d + G * d].view(T, G, d), None, 1e-5)
    pv = 0.7 * src[:, H * d + G * d : H * d + G * d + G * e] + 0.3 * v_first[:, : G * e]
    want = plain_sigmoid_attention(pq, pk, pv.view(T, G, e), 0.4, rel, far, talk, pb) * torch.sigmoid(gate)[:, :, None]
    torch.testing.assert_close(out.view(T, H, e), want, rtol=2e-5, atol=2e-5)
