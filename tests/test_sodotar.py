"""Sodotar without a GPU: the reader of ``config.json``, the layout it gives, the plain mechanisms on hand-made
cases, and the new kernels' plain twins against the plain mechanisms."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from fastgen_amd.config import ConfigError, get_architecture
from fastgen_amd.engine.model import build_parts
from fastgen_amd.kernels import ops, twins
from plain_sodotar import (ODD, PAIR, WIDE, plain_block_mask, plain_diff_attention, plain_expert, plain_forward,
                           plain_rms, plain_rotate, plain_route, plain_softmax_rows, plain_streams_step, plain_weights)


def test_the_reader_round_trips_and_names_missing_keys():
    arch = get_architecture(PAIR)
    assert arch.name == "Sodotar"
    for config in (PAIR, ODD, WIDE):
        args = arch.parse(config)
        assert arch.parse(arch.to_hf_config(args)) == args
    broken = copy.deepcopy(PAIR)
    del broken["layers"][1]["mixer"]["kv_rank"]
    with pytest.raises(ConfigError, match="kv_rank"):
        arch.parse(broken)
    broken = copy.deepcopy(PAIR)
    broken["layers"][2]["mixer"]["kv_from"] = 1  # a latent layer has no keys of that kind
    with pytest.raises(ConfigError, match="kv_from"):
        arch.parse(broken)
    broken = copy.deepcopy(PAIR)
    broken["layers"][0]["mlp"]["router"]["top"] = 7
    with pytest.raises(ConfigError, match="top"):
        arch.parse(broken)


def test_the_layout_names_every_tensor_of_the_checkpoint_and_shares_the_cache():
    arch = get_architecture(PAIR)
    for config in (PAIR, WIDE):
        layout = arch.layout(arch.parse(config))
        names = {s.name: tuple(s.shape) for s in build_parts(layout).tensor_specs()}
        weights = plain_weights(config, 0)
        assert names == {k: tuple(v.shape) for k, v in weights.items()}
    layout = arch.layout(arch.parse(PAIR))
    assert layout.streams == 2 and layout.order[2].reads_cache_of == 0 and layout.order[1].reads_cache_of is None
    # one stream and no tensors for it: the arrangement's weights are ones, nothing is asked of the checkpoint
    one = copy.deepcopy(ODD)
    layout = arch.layout(arch.parse(one))
    assert not any(".hc" in s.name for s in build_parts(layout).tensor_specs())
    layout = arch.layout(arch.parse(one, lambda name: (1,) if name == "l0.hc1.in" else None))
    assert any(".hc" in s.name for s in build_parts(layout).tensor_specs())


def test_block_mask_and_rotation_by_hand():
    m = plain_block_mask(7, 3)
    assert m[2].tolist() == [True, True, True, False, False, False, False]
    assert m[3].tolist() == [False, False, False, True, False, False, False]
    assert m[6].tolist() == [False] * 6 + [True]
    assert plain_block_mask(4, None)[3].tolist() == [True] * 4
    # the engine's encoding of the same mask: the first key a position sees
    for size in (1, 3, 16):
        for p in range(40):
            lo = p - p % size
            assert plain_block_mask(p + 1, size)[p].nonzero().flatten().tolist() == list(range(lo, p + 1))
    x = torch.zeros(3, 1, 6)
    x[:, 0, 0] = 1.0  # dimension 0 pairs with dimension 2 of a run of 4; dimensions 4, 5 pass
    x[:, 0, 5] = 7.0
    y = plain_rotate(x, 100.0, 4)
    for p in range(3):
        assert torch.allclose(y[p, 0], torch.tensor([math.cos(p), 0.0, math.sin(p), 0.0, 0.0, 7.0]), atol=1e-6)
    y = plain_rotate(x, 100.0, 2, first=4)  # a run that starts behind the plain part
    assert torch.allclose(y[2, 0, 4:], torch.tensor([-7.0 * math.sin(2.0), 7.0 * math.cos(2.0)]), atol=1e-5)


def test_sink_and_softmax_by_hand():
    s = torch.tensor([[[0.0, 0.0], [math.log(2.0), 0.0]]])
    vis = plain_block_mask(2, None)
    a = plain_softmax_rows(s, vis, torch.tensor([0.0]))
    assert torch.allclose(a[0, 0], torch.tensor([0.5, 0.0]))  # one key and the sink, equal scores
    assert torch.allclose(a[0, 1], torch.tensor([0.5, 0.25]))  # 2 : 1 : 1 (sink)
    a = plain_softmax_rows(s, vis)
    assert torch.allclose(a[0, 1], torch.tensor([2 / 3, 1 / 3]))


def test_differential_attention_by_hand():
    """One head, one token: both maps put all weight on the one key, so o = (1 - lam) v, normed, times 1 - c."""
    d, e, D = 4, 6, 8
    g = torch.Generator().manual_seed(0)
    w = {"p.q": torch.randn(2 * d, D, generator=g), "p.k": torch.randn(2 * d, D, generator=g), "p.v": torch.randn(e, D, generator=g),
         "p.o": torch.eye(e), "p.lq1": torch.full((d,), 0.5), "p.lk1": torch.full((d,), 0.5), "p.lq2": torch.zeros(d),
         "p.lk2": torch.ones(d)}
    m = {"heads": 1, "kv_heads": 1, "dim": d, "vdim": e, "scale": 0.5, "diff": 0.25, "rot": {"base": 10.0, "dims": 2}}
    x = torch.randn(1, D, generator=g)
    y, _ = plain_diff_attention(x, w, "p", m, 1e-6, torch.float32)
    lam = math.exp(1.0) - 1.0 + 0.25
    v = x @ w["p.v"].T
    want = plain_rms((1 - lam) * v, None, 1e-6) * 0.75
    assert torch.allclose(y, want, atol=1e-5)
    # the twin of the kernel that takes the difference: heads of a group lie as [map 1 of its heads | map 2 ...]
    att = torch.randn(3, 2 * 4 * 8, generator=g)
    out = torch.zeros(3, 4 * 6)
    twins.head_diff_norm(att, 8, out, 4, 2, 6, lam, 1e-6, 0.75)
    a = att.view(3, 8, 8)
    for h, (i1, i2) in enumerate(((0, 2), (1, 3), (4, 6), (5, 7))):
        o = a[:, i1, :6] - lam * a[:, i2, :6]
        assert torch.allclose(out[:, h * 6 : (h + 1) * 6], plain_rms(o, None, 1e-6) * 0.75, atol=1e-5)


def test_routing_and_the_limited_activation_by_hand():
    x = torch.eye(3)
    router = torch.tensor([[2.0, 0.0, 0.0], [1.0, 0.0, 5.0], [0.0, 0.0, 5.0], [0.5, 0.0, 0.0]])
    corr = torch.tensor([0.0, 0.0, 0.0, 0.9])
    chosen, ws = plain_route(x, router, corr, 2, torch.float32)
    s = torch.softmax(torch.tensor([2.0, 1.0, 0.0, 0.5]), 0)
    assert chosen[0].tolist() == [3, 0]  # the correction lifts expert 3 over expert 0 for the choice alone
    assert torch.allclose(ws[0], torch.stack([s[3], s[0]]) / (s[3] + s[0]))
    assert chosen[1].tolist() == [3, 0]  # equal scores: the correction, then the lower expert
    assert chosen[2].tolist() == [3, 1]  # behind the lifted expert a tie of 1 and 2: the lower one
    ti, tw = twins.moe_route(x, router, None, 2, False, corr, 1, 1, 1.0, True, 0)
    assert torch.equal(ti.long(), chosen) and torch.allclose(tw, ws)
    w = {"e.gate": torch.tensor([[3.0], [-1.0]]), "e.up": torch.tensor([[-9.0], [0.5]]), "e.down": torch.eye(2)}
    y = plain_expert(torch.ones(1, 1), w, "e", 2.0, torch.float32)
    g0, g1 = 2.0, -1.0  # the gate is cut from above only
    want = torch.tensor([[g0 / (1 + math.exp(-1.702 * g0)) * (-2.0 + 1), g1 / (1 + math.exp(1.702)) * 1.5]])
    assert torch.allclose(y, want, atol=1e-6)
    gu = torch.zeros(1, 16)
    gu[0, 0], gu[0, 1], gu[0, 8], gu[0, 9] = 3.0, -1.0, -9.0, 0.5  # gate and up interleaved in groups of 8
    assert torch.allclose(twins.gated_mul(gu, None, "limited", torch.float32, None, 2.0, 1.702)[0, :2], want[0], atol=1e-6)


def test_streams_by_hand_and_the_twin():
    X = torch.stack([torch.full((2, 3), 1.0), torch.full((2, 3), 10.0)])
    w = {"h.in": torch.tensor([1.0, 0.5]), "h.out": torch.tensor([2.0, -1.0]), "h.mix": torch.tensor([[1.0, 3.0], [0.0, 1.0]])}
    new = plain_streams_step(X, w, "h", lambda u: u * 0 + 100.0)  # u = 6; y = 100
    assert torch.allclose(new[0], torch.full((2, 3), 1.0 + 200.0))  # mix[0, 0] x0 + mix[1, 0] x1 + 2 y
    assert torch.allclose(new[1], torch.full((2, 3), 3.0 + 10.0 - 100.0))
    x = X.clone()
    u = torch.empty(2, 3)
    twins.streams_step(x, ops.StreamUpdate(torch.full((2, 3), 100.0), w["h.mix"], w["h.out"]), w["h.in"], None, 0.0, None, None, u)
    assert torch.allclose(x, new) and torch.allclose(u, new[0] + 0.5 * new[1])


def test_a_whole_model_in_float64_and_float32_agree():
    w = plain_weights(PAIR, 3)
    toks = list(range(5, 45))
    a, b = plain_forward(w, PAIR, toks, torch.float64), plain_forward(w, PAIR, toks)
    assert float((a - b.double()).abs().max()) < 1e-3 * float(a.abs().max())
