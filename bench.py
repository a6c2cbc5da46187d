#!/usr/bin/python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]
    python bench.py --workload serve        # continuous batching, see serve_workload()
    python bench.py --workload readme       # the load of the reference's README, see readme_workload()
    python bench.py --workload readme --shape 70b   # the same load at the 70B sizes, cache = the memory left
    python bench.py --workload buderax      # the Buderax design beside the dense Llama at equal sizes
    python bench.py --workload gisodra      # the Gisodra design beside the dense Llama at equal sizes
    python bench.py --workload zudisun      # the Zudisun design beside Gisodra and the dense Llama at equal sizes
    python bench.py --workload sodotar      # the Sodotar design beside Gisodra and the dense Llama at equal sizes

The model has the layer sizes of Llama 3.1 8B (32 layers, hidden 4096, 32
heads, 8 kv heads, head size 128, feed-forward 14336, vocabulary 128256,
llama3 rope scaling) with random bfloat16 weights.  A "step" is one decode
step of a batch whose requests each hold a 2,048-token prompt; ``value`` is
decoded tokens a second.  The same line carries the time of a 2,048-token
prefill, the decode step's fraction of the HBM roofline, and decode at batch
1 and 64.  Token ids are uniform random (synthetic); nothing is read from disk.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM = 8.0e12  # bytes/s, MI355X published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_8B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
    num_attention_heads=32, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=False, max_position_embeddings=131072,
)
PROMPT_LEN = 2048
CONTEXT_LEN = 8192  # capacity per request
PAGE = 64


LLAMA_3B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=3072, intermediate_size=8192, num_hidden_layers=28,
    num_attention_heads=24, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=True, max_position_embeddings=131072,
)


LLAMA_70B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=8192, intermediate_size=28672, num_hidden_layers=80,
    num_attention_heads=64, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=False, max_position_embeddings=131072,
)
SHAPES = {"3b": ("llama-3.2-3b-shape-random", LLAMA_3B), "8b": ("llama-3.1-8b-shape-random", LLAMA_8B),
          "70b": ("llama-3.1-70b-shape-random", LLAMA_70B)}


def workload_roofline(engine, cfg: dict, seconds: float) -> dict:
    """Where a whole run stands against the two rooflines: the bytes its steps had to read (every weight once
    a step, and the cache of every request in the step) over the time and the HBM peak; the flops of its matrix
    products and attention over the time and the bf16 MFMA peak.  A run is bound by neither alone (its prompt
    steps by the matrix cores, its decode steps by memory), so the two fractions together say how much of the
    GPU it used."""
    D, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    H, KV, L = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["num_hidden_layers"]
    hd = D // H
    layer_params = D * (H + 2 * KV) * hd + H * hd * D + 3 * D * F
    w = engine.work
    weight_bytes = (L * layer_params + D * V) * 2
    nbytes = w.steps * weight_bytes + w.cache_reads * 2 * KV * hd * 2 * L
    flops = 2 * w.tokens * L * layer_params + 4 * H * hd * L * w.keys_attended
    return {"hbm_frac": round(nbytes / seconds / PEAK_HBM, 4), "mfma_frac": round(flops / seconds / PEAK_FLOPS["bf16"], 4),
            "gbytes": round(nbytes / 1e9, 1), "tflop": round(flops / 1e12, 1), "steps": w.steps, "tokens": w.tokens}


def serve_workload(n_requests: int = 256, step_budget: int = 2048, shape: str = "3b") -> int:
    """Continuous batching at the Llama 3.2 3B shape (random bfloat16 weights): ``n_requests`` requests
    arrive at once, prompts of 128..4096 uniform random ids, 32..512 greedy tokens each, at most 256 live,
    a budget of ``step_budget`` tokens a step (prompt portions beside decoded tokens).  One JSON line: generated
    tokens a second over the whole run, prompt processing included."""
    import random

    import torch

    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    rng = random.Random(3)
    plens = [rng.randint(128, 4096) for _ in range(n_requests)]
    olens = [rng.randint(32, 512) for _ in range(n_requests)]
    max_batch = min(256, n_requests)
    model_name, cfg = SHAPES[shape]
    engine = Engine.from_config(cfg, seed=3, dtype=torch.bfloat16, page_size=PAGE, max_tokens=max_batch * 4672,
                                max_batch=max_batch, max_step_tokens=step_budget)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in plens]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for p, o in zip(prompts, olens):
        engine.add_request(p, SamplingParams(temperature=0.0, max_new_tokens=o))
    n_done, last = 0, t0
    while engine.has_work():
        n_done += len(engine.step())
        if time.perf_counter() - last > 20:
            last = time.perf_counter()
            print(f"[bench] {n_done}/{n_requests} requests done", file=sys.stderr, flush=True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    print(json.dumps({
        "metric": "generated tok/s, continuous batching", "value": round(sum(olens) / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "seconds": round(dt, 3), "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
        "roofline": workload_roofline(engine, cfg, dt),
        "config": {"model": model_name, "requests": n_requests, "prompt_tokens": sum(plens),
                   "generated_tokens": sum(olens), "max_batch": max_batch, "step_budget": step_budget, "page_size": PAGE,
                   "engine_steps": engine.n_steps, "preemptions": engine.scheduler.n_preemptions,
                   "weight_copies": 2 if engine.model.packed() else 1},
    }), flush=True)
    return 0


def readme_workload(shape: str = "8b") -> int:
    """The load behind the numbers of the reference's README (``README.md:22-28``, ``scripts/bench.py:104-106``:
    512 prompts of 1,024 tokens, 128 decode steps each, generated tokens over the wall-clock time of the whole
    batch), with random bfloat16 weights and uniform random ids, at the Llama 3.1 8B shape or, ``--shape 70b``, at
    the 70B shape (141 GB of weights).  The cache is what the GPU has free once the weights are in place
    (``fastgen/utils/tune.py:68-84`` sizes it from a budget): at 8B it holds all 512 requests, at 70B it does not
    and requests are preempted and recomputed.  The reference publishes 3,430 tok/s for Mistral 7B on one H100 and
    2,260 tok/s for Llama 70B on eight, through its server: other models and other hardware, so the ratio in
    ``vs_published`` is context, not a like-for-like comparison."""
    import torch

    from fastgen_amd.engine import Engine, Model
    from fastgen_amd.sampling import SamplingParams

    n, p_len, n_gen, max_batch = 512, 1024, 128, 512
    model_name, cfg = SHAPES[shape]
    published = {"8b": (3430.0, "3430 tok/s, Mistral 7B, 1x H100 (reference README)"),
                 "70b": (2260.0, "2260 tok/s, Llama 70B, 8x H100 (reference README)")}.get(shape)
    t0 = time.perf_counter()
    model = Model.random(cfg, 4 if shape == "70b" else 2, torch.bfloat16, "cuda:0")
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    # no request is longer than prompt + generated: the cache never needs more than that for each
    engine = Engine(model, page_size=PAGE, max_tokens=None, max_batch=max_batch, max_step_tokens=8192,
                    max_seq=-(-(p_len + n_gen) // PAGE) * PAGE)
    pool = engine.scheduler.pool_tokens
    print(f"[bench] cache of {pool} tokens ({pool * engine.runner.storage.bytes_per_token() / 1e9:.1f} GB)",
          file=sys.stderr, flush=True)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, cfg["vocab_size"], (p_len,), generator=g).tolist() for _ in range(n)]
    params = SamplingParams(temperature=0.0, max_new_tokens=n_gen)
    torch.cuda.synchronize()
    t0 = last = time.perf_counter()
    for p in prompts:
        engine.add_request(p, params)
    generated = n_done = 0
    while engine.has_work():
        for r in engine.step():
            generated += len(r.generated)
            n_done += 1
        if time.perf_counter() - last > 20:
            last = time.perf_counter()
            print(f"[bench] {n_done}/{n} requests done, {engine.scheduler.n_preemptions} preemptions",
                  file=sys.stderr, flush=True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    print(json.dumps({
        "metric": "generated tok/s, 512 prompts x 1024 tokens, 128 decode steps", "value": round(generated / dt, 1),
        "unit": "tokens/s", "n_gpus": 1, "seconds": round(dt, 3), "higher_is_better": True, "dtype": "bf16",
        "data": "synthetic", "vs_published": round(generated / dt / published[0], 3) if published else None,
        "roofline": workload_roofline(engine, cfg, dt),
        "config": {"model": model_name, "requests": n, "prompt_len": p_len, "generated": n_gen,
                   "max_batch": max_batch, "step_budget": 8192, "page_size": PAGE, "engine_steps": engine.n_steps,
                   "cache_tokens": pool, "cache": "free memory after the weights",
                   "preemptions": engine.scheduler.n_preemptions,
                   "weight_copies": 2 if engine.model.packed() else 1,
                   "published": published[1] if published else None},
    }), flush=True)
    return 0


# Buderax at sizes that resemble a real model's layers; the dense Llama beside it has the same width, heads,
# head size and number of layer runs, and a feed-forward as wide as the experts a token uses (top x ff).
BUDERAX_SIZES = {
    "w1024": dict(width=1024, heads=16, kv_heads=4, dim=64, experts=16, top=2, ff=512, layers=6,
                  loop=dict(start=2, stop=4, times=2), vocab=32000),
    "w2048": dict(width=2048, heads=16, kv_heads=4, dim=128, experts=32, top=4, ff=768, layers=8, loop=None, vocab=32000),
}


def _buderax_configs(z: dict):
    mixer = dict(heads=z["heads"], kv_heads=z["kv_heads"], dim=z["dim"], vdim=z["dim"], scale=z["dim"] ** -0.5,
                 rot=dict(base=1000000.0, dims=z["dim"] // 2, scaling=dict(factor=8.0)))
    mlp = dict(kind="moe", router=dict(experts=z["experts"], top=z["top"]), expert=dict(ff=z["ff"]))
    new = dict(architecture="Buderax", width=z["width"], vocab=z["vocab"], embedding=dict(scale=2.0), norm=dict(eps=1e-6),
               layers=[dict(type="attention", mixer=mixer, mlp=mlp) for _ in range(z["layers"])])
    runs = z["layers"]
    if z["loop"]:
        new["loop"] = z["loop"]
        runs += (z["loop"]["stop"] - z["loop"]["start"]) * (z["loop"]["times"] - 1)
    dense = dict(architectures=["LlamaForCausalLM"], hidden_size=z["width"], intermediate_size=z["top"] * z["ff"],
                 num_hidden_layers=runs, num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"],
                 rms_norm_eps=1e-6, vocab_size=z["vocab"], rope_theta=500000.0, rope_scaling=None,
                 tie_word_embeddings=False, max_position_embeddings=131072)
    return new, dense, runs


def _time(fn, repeats: int = 20) -> float:
    """Seconds of one call: the best of ``repeats`` after three unmeasured ones."""
    import torch

    for _ in range(3):
        fn()
    best = float("inf")
    for _ in range(repeats):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        best = min(best, a.elapsed_time(b) * 1e-3)
    return best


def _buderax_kernels(z: dict, rows: int) -> dict:
    """The routed feed-forward's kernels at ``rows`` tokens beside the dense feed-forward's products with
    the same rows and as many channels a token (top x ff): seconds, and the share of the roofline that
    bounds them (matrix cores for many rows, memory for few: bytes = the matrices read once; of the
    experts, those that the rows can reach)."""
    import torch

    from fastgen_amd.kernels import ops
    from fastgen_amd.kernels.linear import linear

    D, E, top, F = z["width"], z["experts"], z["top"], z["ff"]
    g = torch.Generator(device="cuda").manual_seed(rows)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device="cuda") * 0.05).to(torch.bfloat16)
    x = rnd(rows, D) * 20
    router, bias = rnd(E, D).float(), rnd(E).float()
    wg, wu, wd = rnd(E, F, D), rnd(E, F, D), rnd(E, D, F)
    per_expert = rows * top / E
    tile_rows = next((r for r, least in ((256, 768), (128, 96), (64, 48), (32, 24)) if per_expert >= least), 16)
    choice, weight = ops.moe_route(x, router, bias, top)
    sorted_, tiles = ops.moe_sort(choice, E, tile_rows)
    act = ops.moe_gate_up(x, wg, wu, sorted_, tiles, top, tile_rows)
    y = ops.moe_down(act, wd, sorted_, tiles, tile_rows)
    dense_gu = ops.interleave_gate_up(rnd(top * F, D), rnd(top * F, D))
    dense_d = rnd(D, top * F)
    dense_act = linear(x, dense_gu, epilogue="silu_mul")
    reached = min(E, rows * top)
    flops_gu, flops_d = 2 * rows * top * 2 * F * D, 2 * rows * top * F * D
    out = {}
    for name, fn, flops, nbytes in (
        ("moe_route", lambda: ops.moe_route(x, router, bias, top), 2 * rows * E * D, E * D * 4 + rows * D * 2),
        ("moe_sort", lambda: ops.moe_sort(choice, E, tile_rows), 0, rows * top * 8),
        ("moe_gate_up", lambda: ops.moe_gate_up(x, wg, wu, sorted_, tiles, top, tile_rows), flops_gu, reached * 2 * F * D * 2),
        ("dense_gate_up", lambda: linear(x, dense_gu, epilogue="silu_mul"), flops_gu, top * 2 * F * D * 2),
        ("moe_down", lambda: ops.moe_down(act, wd, sorted_, tiles, tile_rows), flops_d, reached * F * D * 2),
        ("dense_down", lambda: linear(dense_act, dense_d), flops_d, top * F * D * 2),
        ("moe_combine", lambda: ops.moe_combine(y, weight, None), 0, rows * top * D * 4 + rows * D * 4),
    ):
        t = _time(fn)
        out[name] = {"us": round(t * 1e6, 1), "mfma_frac": round(flops / t / PEAK_FLOPS["bf16"], 4),
                     "hbm_frac": round(nbytes / t / PEAK_HBM, 4)}
    return out


def buderax_workload(prefill_tokens: int = 2048, batch: int = 8, context: int = 1024, steps: int = 32, warmup: int = 8) -> int:
    """Prefill and decode throughput of Buderax models with random bfloat16 weights beside dense Llama
    models of equal sizes, and the routed feed-forward's kernels beside the dense feed-forward's.  One JSON line."""
    import torch

    from fastgen_amd.engine import Engine

    results = {}
    for name, z in BUDERAX_SIZES.items():
        new, dense, runs = _buderax_configs(z)
        row = {"layer_runs": runs}
        for label, cfg in (("buderax", new), ("llama", dense)):
            engine = Engine.from_config(cfg, seed=5, dtype=torch.bfloat16, page_size=PAGE,
                                        max_tokens=max(batch * (context + 256), prefill_tokens + PAGE), max_batch=batch,
                                        max_step_tokens=prefill_tokens)
            g = torch.Generator().manual_seed(0)
            prompt = lambda n: torch.randint(0, z["vocab"], (n,), generator=g).tolist()
            pre = min(engine.time_prefill(prompt(prefill_tokens), repeats=5))
            dt = engine.time_decode([prompt(context) for _ in range(batch)], steps=steps, warmup=warmup)
            row[label] = {"prefill_tok_s": round(prefill_tokens / pre, 1), "prefill_ms": round(pre * 1e3, 3),
                          "decode_tok_s": round(batch * steps / dt, 1), "decode_ms_per_step": round(dt / steps * 1e3, 4),
                          "weights_gb": round(engine.model.weight_bytes() / 1e9, 3)}
            print(f"[bench] {name} {label}: {row[label]}", file=sys.stderr, flush=True)
            del engine
            torch.cuda.empty_cache()
        row["kernels_prefill"] = _buderax_kernels(z, prefill_tokens)
        row["kernels_decode"] = _buderax_kernels(z, batch)
        print(f"[bench] {name} kernels: {row['kernels_prefill']} {row['kernels_decode']}", file=sys.stderr, flush=True)
        results[name] = row
    first = results[next(iter(results))]
    print(json.dumps({
        "metric": "Buderax beside the dense Llama at equal sizes: prefill and decode tok/s", "unit": "tokens/s",
        "value": first["buderax"]["decode_tok_s"], "n_gpus": 1, "steps": steps, "warmup": warmup, "higher_is_better": True,
        "dtype": "bf16", "data": "synthetic",
        "config": {"prefill_tokens": prefill_tokens, "decode_batch": batch, "decode_context": context, "page_size": PAGE,
                   "sizes": BUDERAX_SIZES},
        "results": results,
    }), flush=True)
    return 0


# Gisodra at sizes that resemble a real model's layers: eight layers in the order attention, gated linear
# attention, attention on the first one's cache, latent attention, twice; the dense Llama beside it has the same
# width, heads, head size, feed-forward width and number of layers.
GISODRA_SIZES = {
    "w1024": dict(width=1024, heads=16, kv_heads=4, dim=64, ff=2816, window=1024, gla_heads=8, gla_dim=64, gla_vdim=128,
                  lat_dim=64, rot_dim=32, kv_rank=192, q_rank=384, vocab=32000),
    "w2048": dict(width=2048, heads=16, kv_heads=4, dim=128, ff=5632, window=4096, gla_heads=16, gla_dim=128, gla_vdim=128,
                  lat_dim=128, rot_dim=64, kv_rank=192, q_rank=768, vocab=32000),
}


def _gisodra_configs(z: dict):
    attn = lambda **more: dict(type="attention", mlp=dict(kind="dense", ff=z["ff"]), mixer=dict(
        heads=z["heads"], kv_heads=z["kv_heads"], dim=z["dim"], vdim=z["dim"], scale=z["dim"] ** -0.5,
        mask=dict(size=z["window"]), **more))
    gla = dict(type="gla", mlp=None, mixer=dict(heads=z["gla_heads"], dim=z["gla_dim"], vdim=z["gla_vdim"], tau=16.0))
    latent = dict(type="latent_attention", mlp=dict(kind="dense", ff=z["ff"]), mixer=dict(
        heads=z["heads"], dim=z["lat_dim"], rot_dim=z["rot_dim"], vdim=z["dim"], kv_rank=z["kv_rank"], q_rank=z["q_rank"],
        scale=(z["lat_dim"] + z["rot_dim"]) ** -0.5, mask=dict(size=z["window"]), rot=dict(base=1000000.0, dims=z["rot_dim"])))
    layers = [attn(), gla, attn(kv_from=0), latent, attn(), gla, attn(kv_from=4), latent]
    new = dict(architecture="Gisodra", width=z["width"], vocab=z["vocab"], norm=dict(eps=1e-6), logit_softcap=30.0, layers=layers)
    dense = dict(architectures=["LlamaForCausalLM"], hidden_size=z["width"], intermediate_size=z["ff"],
                 num_hidden_layers=len(layers), num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"],
                 rms_norm_eps=1e-6, vocab_size=z["vocab"], rope_theta=500000.0, rope_scaling=None,
                 tie_word_embeddings=True, max_position_embeddings=131072)
    return new, dense


def _gisodra_kernels(z: dict, rows: int, context: int) -> dict:
    """The design's own kernels at ``rows`` tokens (one prompt of ``rows`` tokens, or ``rows`` sequences of one
    token at ``context`` cached ones), each beside the like kernel of the dense decoder on operands of the same
    size: microseconds, and the shares of the memory roofline (the bytes the kernel has to move) and of the
    matrix cores' (its products' flops)."""
    import torch

    from fastgen_amd.kernels import ops
    from fastgen_amd.kernels.linear import linear

    D, H, G, d, P = z["width"], z["heads"], z["kv_heads"], z["dim"], PAGE
    R, r, dl, Q = z["kv_rank"], z["rot_dim"], z["lat_dim"], z["q_rank"]
    gh, gd, ge = z["gla_heads"], z["gla_dim"], z["gla_vdim"]
    g = torch.Generator(device="cuda").manual_seed(rows)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device="cuda") * 0.05).to(torch.bfloat16)
    f32 = lambda *shape: torch.randn(*shape, generator=g, device="cuda")
    decode = rows <= 16
    n_seqs = rows if decode else 1
    n_pages = rows // P + 2
    slots = torch.arange(rows, dtype=torch.int32, device="cuda")
    table = ops.rope_table(torch.arange(rows, dtype=torch.int32, device="cuda"), f32(max(d, r) // 2).abs())
    out = {}

    def put(name, fn, nbytes, flops=0):
        t = _time(fn)
        out[name] = {"us": round(t * 1e6, 1), "hbm_frac": round(nbytes / t / PEAK_HBM, 4),
                     "mfma_frac": round(flops / t / PEAK_FLOPS["bf16"], 4)}

    # between the q/k/v product and the attention: bias, norms per head, cache write; beside rotation and cache write
    qkv32, qkv16 = f32(rows, (H + 2 * G) * d), rnd(rows, (H + 2 * G) * d)
    bias, nw = f32((H + 2 * G) * d), f32(d)
    kp, vp = rnd(n_pages, G, P, d), rnd(n_pages, G, d, P)
    q_out = torch.empty(rows, H * d, dtype=torch.bfloat16, device="cuda")
    put("heads_prepare (attention)", lambda: ops.heads_prepare(
        qkv32, bias, 1e-6, n_q=H, q_col=0, q_width=d, q_norm=nw, q_norm_dims=d, q_out=q_out, q_out_width=d, n_kv=G,
        k_col=H * d, k_width=d, k_norm=nw, k_norm_dims=d, v_col=(H + G) * d, v_width=d, slots=slots, k_pages=kp, v_pages=vp),
        qkv32.numel() * 4 + (H + 2 * G) * d * rows * 2)
    table_d = table[:, : d // 2].contiguous()
    put("rope_kv_write (llama)", lambda: ops.rope_kv_write(qkv16, slots, None, slots, kp, vp, H, G, d, d, table=table_d),
        qkv16.numel() * 2 + (H + 2 * G) * d * rows * 2)
    # the norms around a sublayer; beside the one norm of the dense decoder
    h, delta, w1, w2 = f32(rows, D), rnd(rows, D), rnd(D), rnd(D)
    normed = torch.empty(rows, D, dtype=torch.bfloat16, device="cuda")
    put("post_add_rmsnorm", lambda: ops.post_add_rmsnorm(h, delta, w1, 1e-6, w2, 1e-6, normed), rows * D * (4 + 4 + 2 + 2))
    put("add_rmsnorm (llama)", lambda: ops.add_rmsnorm(h, delta, w2, 1e-6, normed), rows * D * (4 + 4 + 2 + 2))
    # the feed-forward's first product with its activation
    x, wgu = rnd(rows, D) * 20, ops.interleave_gate_up(rnd(z["ff"], D), rnd(z["ff"], D))
    put("gate/up + gelu_tanh", lambda: linear(x, wgu, epilogue="gelu_tanh_mul"), wgu.numel() * 2, 2 * rows * wgu.numel())
    put("gate/up + silu (llama)", lambda: linear(x, wgu, epilogue="silu_mul"), wgu.numel() * 2, 2 * rows * wgu.numel())
    # latent attention: the products per head beside one product of the same flops and weights
    hc = -(-(R + r) // 16) * 16
    q, w_uk_t = rnd(rows, H * (dl + r)), rnd(H, R, dl)
    q_lat = torch.empty(rows, H * hc, dtype=torch.bfloat16, device="cuda")
    put("head_linear (queries into the latent)", lambda: ops.head_linear(q, dl + r, w_uk_t, q_lat, hc, tail=r),
        w_uk_t.numel() * 2 + q.numel() * 2 + q_lat.numel() * 2, 2 * rows * H * R * dl)
    lat, w_uv, gate = rnd(rows, H * hc), rnd(H, d, R), f32(rows, H)
    v_out = torch.empty(rows, H * d, dtype=torch.bfloat16, device="cuda")
    put("head_linear (outputs out of the latent)", lambda: ops.head_linear(lat, hc, w_uv, v_out, d, gate=gate),
        w_uv.numel() * 2 + lat.numel() * 2 + v_out.numel() * 2, 2 * rows * H * R * d)
    xs, wl = rnd(rows, dl), rnd(H * R, dl)
    put("one product of the same flops (library or own)", lambda: linear(xs, wl), wl.numel() * 2 + rows * (dl + H * R) * 2,
        2 * rows * H * R * dl)
    rows32 = f32(rows, Q + R + r + H)
    cq = torch.empty(rows, Q, dtype=torch.bfloat16, device="cuda")
    kl, vl = rnd(n_pages, 1, P, hc), rnd(n_pages, 1, hc, P)
    nq, nk, table_r = f32(Q), f32(R), table[:, : r // 2].contiguous()
    put("heads_prepare (latents)", lambda: ops.heads_prepare(
        rows32, None, 1e-6, n_q=1, q_col=0, q_width=Q, q_norm=nq, q_norm_dims=Q, q_out=cq, q_out_width=Q, n_kv=1, k_col=Q,
        k_width=R + r, k_norm=nk, k_norm_dims=R, v_col=-1, v_width=R, table=table_r, rot_start=R,
        rotary_dim=r, rotate_q=False, slots=slots, k_pages=kl, v_pages=vl), rows * ((Q + R + r) * 4 + Q * 2 + 2 * hc * 2))
    # the recurrence: fp32 vector arithmetic, token by token; four flops a state element and token
    width = 2 * gh * gd + 2 * gh * ge
    rows16, zz, zb = rnd(rows, width), f32(rows, gh * gd), f32(gh * gd)
    state = torch.zeros(n_seqs + 1, gh, gd, ge, device="cuda")
    slot_ids = torch.arange(n_seqs, dtype=torch.int32, device="cuda")
    q_start = torch.arange(0, rows + 1, rows // n_seqs, dtype=torch.int32, device="cuda")
    o32 = torch.empty(rows, gh * ge, device="cuda")
    q_start_host = q_start.cpu().numpy()  # (with it, long runs of tokens are scanned in chunks side by side)
    t = _time(lambda: ops.decay_scan(rows16, 0, gh * gd, 2 * gh * gd, zz, zb, 16.0, gd ** -0.5, state, slot_ids, q_start, n_seqs,
                                     o32, q_start_host=q_start_host))
    if not decode:
        t_chain = _time(lambda: ops.decay_scan(rows16, 0, gh * gd, 2 * gh * gd, zz, zb, 16.0, gd ** -0.5, state, slot_ids, q_start,
                                               n_seqs, o32))
        out["decay_scan, token by token"] = {"us": round(t_chain * 1e6, 1)}
    out["decay_scan"] = {"us": round(t * 1e6, 1),
                         "hbm_frac": round((2 * n_seqs * gh * gd * ge * 4 + rows * (width * 2 + gh * gd * 4 + gh * ge * 4)) / t / PEAK_HBM, 4),
                         "fp32_vector_frac": round(4 * rows * gh * gd * ge / t / 157e12, 4)}
    gated = torch.empty(rows, gh * ge, dtype=torch.bfloat16, device="cuda")
    ng = f32(ge)
    put("head_norm_gate", lambda: ops.head_norm_gate(o32, ng, 1e-6, rows16[:, 2 * gh * gd + gh * ge:], gh, gated),
        rows * gh * ge * (4 + 2 + 2))
    return out


def gisodra_workload(prefill_tokens: int = 2048, batch: int = 8, context: int = 1024, steps: int = 32, warmup: int = 8) -> int:
    """Prefill and decode throughput of Gisodra models with random bfloat16 weights beside dense Llama models
    of equal sizes, and the design's own kernels beside the dense decoder's like ones.  One JSON line."""
    import torch

    from fastgen_amd.engine import Engine

    results = {}
    for name, z in GISODRA_SIZES.items():
        new, dense = _gisodra_configs(z)
        row = {"layers": len(new["layers"])}
        for label, cfg in (("gisodra", new), ("llama", dense)):
            engine = Engine.from_config(cfg, seed=5, dtype=torch.bfloat16, page_size=PAGE,
                                        max_tokens=max(batch * (context + 256), prefill_tokens + PAGE), max_batch=batch,
                                        max_step_tokens=prefill_tokens)
            g = torch.Generator().manual_seed(0)
            prompt = lambda n: torch.randint(0, z["vocab"], (n,), generator=g).tolist()
            pre = min(engine.time_prefill(prompt(prefill_tokens), repeats=5))
            dt = engine.time_decode([prompt(context) for _ in range(batch)], steps=steps, warmup=warmup)
            row[label] = {"prefill_tok_s": round(prefill_tokens / pre, 1), "prefill_ms": round(pre * 1e3, 3),
                          "decode_tok_s": round(batch * steps / dt, 1), "decode_ms_per_step": round(dt / steps * 1e3, 4),
                          "weights_gb": round(engine.model.weight_bytes() / 1e9, 3)}
            print(f"[bench] {name} {label}: {row[label]}", file=sys.stderr, flush=True)
            del engine
            torch.cuda.empty_cache()
        row["kernels_prefill"] = _gisodra_kernels(z, prefill_tokens, context)
        row["kernels_decode"] = _gisodra_kernels(z, batch, context)
        print(f"[bench] {name} kernels: {row['kernels_prefill']} {row['kernels_decode']}", file=sys.stderr, flush=True)
        results[name] = row
    first = results[next(iter(results))]
    print(json.dumps({
        "metric": "Gisodra beside the dense Llama at equal sizes: prefill and decode tok/s", "unit": "tokens/s",
        "value": first["gisodra"]["decode_tok_s"], "n_gpus": 1, "steps": steps, "warmup": warmup, "higher_is_better": True,
        "dtype": "bf16", "data": "synthetic",
        "config": {"prefill_tokens": prefill_tokens, "decode_batch": batch, "decode_context": context, "page_size": PAGE,
                   "sizes": GISODRA_SIZES},
        "results": results,
    }), flush=True)
    return 0


# Zudisun at sizes that resemble a real model's layers: eight layers in the order sigmoid attention with a dense
# feed-forward, selective scan with a routed one, selective scan with a dense one, sigmoid attention with a routed
# one, twice.  Beside it: Gisodra (the framework's other design with attention and recurrent layers side by side)
# and the dense Llama, both of the same width, heads, head size, dense feed-forward width and number of layers.
ZUDISUN_SIZES = {
    "w1024": dict(width=1024, heads=16, kv_heads=4, dim=64, ff=2816, inner=2048, state=16, dt_rank=64, conv=4,
                  experts=16, top=2, expert_ff=704, groups=4, keep=2, shared_ff=704, far=2048.0, rows=32, vocab=32000),
    "w2048": dict(width=2048, heads=16, kv_heads=4, dim=128, ff=5632, inner=4096, state=16, dt_rank=128, conv=4,
                  experts=32, top=4, expert_ff=768, groups=8, keep=4, shared_ff=1536, far=2048.0, rows=32, vocab=32000),
}


def _zudisun_configs(z: dict):
    attn = lambda mlp: dict(type="attention", mlp=mlp, mixer=dict(
        heads=z["heads"], kv_heads=z["kv_heads"], dim=z["dim"], vdim=z["dim"], scale=z["dim"] ** -0.5,
        q_temp=dict(coef=0.5, every=512), bias_max=z["far"], bias_rows=z["rows"], v_mix=True))
    scan = lambda mlp: dict(type="mamba1", mlp=mlp, mixer=dict(inner=z["inner"], state=z["state"], dt_rank=z["dt_rank"], conv=z["conv"]))
    dense_ff = dict(kind="dense", ff=z["ff"])
    routed = dict(kind="moe", expert=dict(ff=z["expert_ff"]), shared=dict(ff=z["shared_ff"]),
                  router=dict(experts=z["experts"], top=z["top"], scale=1.5, groups=dict(count=z["groups"], keep=z["keep"])))
    layers = [attn(dense_ff), scan(routed), scan(dense_ff), attn(routed)] * 2
    new = dict(architecture="Zudisun", width=z["width"], vocab=z["vocab"], norm=dict(eps=1e-6), layers=layers)
    dense = dict(architectures=["LlamaForCausalLM"], hidden_size=z["width"], intermediate_size=z["ff"],
                 num_hidden_layers=len(layers), num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"],
                 rms_norm_eps=1e-6, vocab_size=z["vocab"], rope_theta=500000.0, rope_scaling=None,
                 tie_word_embeddings=False, max_position_embeddings=131072)
    return new, dense


def _zudisun_kernels(z: dict, rows: int, context: int) -> dict:
    """The design's own kernels at ``rows`` tokens (one prompt of ``rows`` tokens, or ``rows`` sequences of one token
    at ``context`` cached ones), each beside the like kernel of the framework's other models on operands of the
    same size: microseconds, and the shares of the memory roofline (the bytes the kernel has to move), of the
    matrix cores' (its products' flops) and of the fp32 vector units' (the flops that are fp32 by design)."""
    import torch

    from fastgen_amd.kernels import ops
    from fastgen_amd.parts.position import distance_table

    D, H, G, d, P = z["width"], z["heads"], z["kv_heads"], z["dim"], PAGE
    C, N, R, K = z["inner"], z["state"], z["dt_rank"], z["conv"]
    g = torch.Generator(device="cuda").manual_seed(rows)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device="cuda") * 0.05).to(torch.bfloat16)
    f32 = lambda *shape: torch.randn(*shape, generator=g, device="cuda")
    i32 = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    decode = rows <= 64
    n_seqs = rows if decode else 1
    out = {}

    def put(name, fn, nbytes, flops=0, vector_flops=0):
        t = _time(fn)
        out[name] = {"us": round(t * 1e6, 1), "hbm_frac": round(nbytes / t / PEAK_HBM, 4),
                     "mfma_frac": round(flops / t / PEAK_FLOPS["bf16"], 4),
                     "fp32_vector_frac": round(vector_flops / t / PEAK_FLOPS["fp32"], 4)}

    # ---- attention over the pages: a prompt of `rows` tokens, or `rows` sequences of `context` keys each
    per_seq = rows if not decode else context
    pages_per_seq = -(-per_seq // P)
    n_pages = n_seqs * pages_per_seq + 1
    kp, vp = rnd(n_pages, G, P, d), rnd(n_pages, G, d, P)
    table = torch.arange(n_seqs * pages_per_seq, dtype=torch.int32, device="cuda").view(n_seqs, pages_per_seq).contiguous()
    if decode:
        seq_of_token, positions = i32(list(range(rows))), i32([context - 1] * rows)
        pairs = rows * context
    else:
        seq_of_token, positions = i32([0] * rows), i32(list(range(rows)))
        pairs = rows * (rows + 1) // 2
    q, o = rnd(rows, H * d), torch.empty(rows, H * d, dtype=torch.bfloat16, device="cuda")
    rel = distance_table(f32(z["rows"], H), z["far"]).contiguous()
    talk, pb, gate = f32(H, H) / H, f32(H) - 3.0, f32(rows, H)
    split = per_seq if decode else 0
    kv_bytes = (n_seqs * per_seq * 2 * G * d + 2 * rows * H * d) * 2
    # per (query, key) pair: the two products (matrix cores), and in fp32 by design: the heads' mixing (2 H^2), the
    # bias, scale and sigmoid (about 8 a head)
    # bfloat16 runs on the matrix cores, an item of up to 16 tokens of a sequence a workgroup and chunk of keys
    if decode:
        items = [[b, b, 1, context - 1] for b in range(rows)]
    else:
        items, split = ops.sigmoid_attention_items([rows], [0, rows], [0]), rows
    tiles = dict(items=ops.upload(items, torch.int32, "cuda"), mixed=ops.sigmoid_attention_mixed(d ** -0.5, H, rel, talk, pb, "cuda"))
    put("sigmoid_attention", lambda: ops.sigmoid_attention(q, d, o, d, kp, vp, table, seq_of_token, positions, H, d ** -0.5, rel,
                                                           talk, pb, gate, split_for=split, **tiles),
        kv_bytes, 4 * pairs * H * d, pairs * (2 * H * H + 8 * H))
    put("sigmoid_attention, general kernel (what float32 runs)",
        lambda: ops.sigmoid_attention(q, d, o, d, kp, vp, table, seq_of_token, positions, H, d ** -0.5, rel, talk, pb, gate,
                                      split_for=split if decode else 0), kv_bytes, 0, pairs * (4 * H * d + 2 * H * H + 8 * H))
    q_start = i32(list(range(0, rows + 1, rows // n_seqs)))
    put("paged_attention_general (the softmax attention's general kernel)",
        lambda: ops.paged_attention_general(q, o, kp, vp, table, seq_of_token, positions, H, d ** -0.5), kv_bytes, 4 * pairs * H * d)
    # ---- between the q/k/v product and the attention: unit norms, temperature, blended values, cache write
    width = (H + 2 * G) * d + H
    rows32, v_first = f32(rows, width), f32(rows, G * d)
    slots = torch.arange(rows, dtype=torch.int32, device="cuda") if not decode else i32([b * pages_per_seq * P + context - 1 for b in range(rows)])
    put("heads_prepare (unit norms, temperature, blend)", lambda: ops.heads_prepare(
        rows32, None, 1e-6, n_q=H, q_col=0, q_width=d, q_norm_dims=d, q_out=q, q_out_width=d, n_kv=G, k_col=H * d, k_width=d,
        k_norm_dims=d, v_col=(H + G) * d, v_width=d, slots=slots, k_pages=kp, v_pages=vp, norm_plain=True, positions=positions,
        q_temp_coef=0.5, q_temp_every=512, v_first=v_first, v_blend=0.3), rows * (width * 4 + G * d * 4 + (H + 2 * G) * d * 2))
    nw = f32(d)
    put("heads_prepare (gisodra: norms with weights)", lambda: ops.heads_prepare(
        rows32, None, 1e-6, n_q=H, q_col=0, q_width=d, q_norm=nw, q_norm_dims=d, q_out=q, q_out_width=d, n_kv=G, k_col=H * d,
        k_width=d, k_norm=nw, k_norm_dims=d, v_col=(H + G) * d, v_width=d, slots=slots, k_pages=kp, v_pages=vp),
        rows * (width * 4 + (H + 2 * G) * d * 2))
    # ---- the selective scan and its convolution; beside Gisodra's recurrence with a state of the same size
    xz, dt = rnd(rows, 2 * C), f32(rows, C)
    narrow = rnd(rows, -(-(R + 2 * N) // 8) * 8)
    taps, cb, db, A, Dk = f32(C, K), f32(C), f32(C) - 2.0, -f32(C, N).abs() - 0.1, f32(C)
    state = torch.zeros(n_seqs + 1, C, N + K - 1, device="cuda")
    slot_ids = torch.arange(n_seqs, dtype=torch.int32, device="cuda")
    seq_rows = i32([t // (rows // n_seqs) for t in range(rows)])
    u, y = torch.empty(rows, C, dtype=torch.bfloat16, device="cuda"), torch.empty(rows, C, dtype=torch.bfloat16, device="cuda")
    put("causal_conv", lambda: ops.causal_conv(xz, taps, cb, state, N, slot_ids, seq_rows, q_start, u, activation="silu"),
        rows * C * 4 + n_seqs * C * (K - 1) * 4, 0, 2 * rows * C * K)
    # per state element and token: a product and an exponential for the decay, two multiply-adds; all fp32 by design
    q_start_host = q_start.cpu().numpy()  # (with it, long runs of tokens are scanned in chunks side by side)
    put("selective_scan", lambda: ops.selective_scan(u, dt, db, A, narrow, R, R + N, Dk, xz[:, C:], xz, K, state, slot_ids, q_start,
                                                     n_seqs, y, q_start_host=q_start_host),
        2 * n_seqs * C * (N + K - 1) * 4 + rows * (C * (2 + 4 + 2 + 2 + 2) + 2 * N * 2), 0, 6 * rows * C * N)
    gh, gd = z["heads"], 64
    ge = C * N // (gh * gd)  # as many state elements as the scan has
    gw = 2 * gh * gd + 2 * gh * ge
    rows16, zz, zb = rnd(rows, gw), f32(rows, gh * gd), f32(gh * gd)
    gstate = torch.zeros(n_seqs + 1, gh, gd, ge, device="cuda")
    o32 = torch.empty(rows, gh * ge, device="cuda")
    t = _time(lambda: ops.decay_scan(rows16, 0, gh * gd, 2 * gh * gd, zz, zb, 16.0, gd ** -0.5, gstate, slot_ids, q_start, n_seqs, o32,
                                     q_start_host=q_start_host))
    out["decay_scan (gisodra, a state of equal size)"] = {
        "us": round(t * 1e6, 1),
        "hbm_frac": round((2 * n_seqs * gh * gd * ge * 4 + rows * (gw * 2 + gh * gd * 4 + gh * ge * 4)) / t / PEAK_HBM, 4),
        "fp32_vector_frac": round(4 * rows * gh * gd * ge / t / PEAK_FLOPS["fp32"], 4)}
    if not decode:
        put("selective_scan, token by token", lambda: ops.selective_scan(u, dt, db, A, narrow, R, R + N, Dk, xz[:, C:], xz, K, state,
                                                                         slot_ids, q_start, n_seqs, y), 0, 0, 6 * rows * C * N)
        t = _time(lambda: ops.decay_scan(rows16, 0, gh * gd, 2 * gh * gd, zz, zb, 16.0, gd ** -0.5, gstate, slot_ids, q_start, n_seqs, o32))
        out["decay_scan (gisodra), token by token"] = {"us": round(t * 1e6, 1),
                                                        "fp32_vector_frac": round(4 * rows * gh * gd * ge / t / PEAK_FLOPS["fp32"], 4)}
    # ---- the dense feed-forward's activation with biases; beside the activation alone
    F = z["ff"]
    gu, b = f32(rows, 2 * F), f32(2 * F)
    put("gated_mul (relu, biases, fp32 rows)", lambda: ops.gated_mul(gu, b, "relu", torch.bfloat16), rows * F * (8 + 2))
    gu16 = rnd(rows, 2 * F)
    put("silu_mul (llama, bf16 rows)", lambda: ops.silu_mul(gu16), rows * F * (4 + 2))
    # ---- the stream's rows with a sublayer's normed output added; beside the dense decoder's norm
    h, delta, w1, w2, ob = f32(rows, D), rnd(rows, D), rnd(D), rnd(D), f32(D)
    normed = torch.empty(rows, D, dtype=torch.bfloat16, device="cuda")
    put("post_add_rmsnorm (rows of the stream, output bias)",
        lambda: ops.post_add_rmsnorm(h, delta, w1, 1e-6, None, 0.0, normed, delta_bias=ob), rows * D * (4 + 4 + 2 + 2))
    put("add_rmsnorm (llama)", lambda: ops.add_rmsnorm(h, delta, w2, 1e-6, normed), rows * D * (4 + 4 + 2 + 2))
    # ---- the router: sigmoid scores, groups, correction; beside the softmax router
    x, wr, corr = rnd(rows, D), f32(z["experts"], D) / 30, f32(z["experts"])
    route_bytes = rows * D * 2 + z["experts"] * D * 4
    put("moe_route (sigmoid, groups)", lambda: ops.moe_route(x, wr, None, z["top"], True, corr, z["groups"], z["keep"], 1.5),
        route_bytes, 0, 2 * rows * D * z["experts"])
    put("moe_route (buderax, softmax)", lambda: ops.moe_route(x, wr, None, z["top"]), route_bytes, 0, 2 * rows * D * z["experts"])
    return out


def zudisun_workload(prefill_tokens: int = 2048, batch: int = 8, context: int = 1024, steps: int = 32, warmup: int = 8) -> int:
    """Prefill and decode throughput of Zudisun models with random bfloat16 weights beside Gisodra and dense Llama
    models of equal sizes, and the design's own kernels beside the other models' like ones.  One JSON line."""
    import torch

    from fastgen_amd.engine import Engine

    results = {}
    for name, z in ZUDISUN_SIZES.items():
        new, dense = _zudisun_configs(z)
        hybrid, _ = _gisodra_configs(GISODRA_SIZES[name])
        row = {"layers": len(new["layers"])}
        for label, cfg in (("zudisun", new), ("gisodra", hybrid), ("llama", dense)):
            engine = Engine.from_config(cfg, seed=5, dtype=torch.bfloat16, page_size=PAGE,
                                        max_tokens=max(batch * (context + 256), prefill_tokens + PAGE), max_batch=batch,
                                        max_step_tokens=prefill_tokens)
            g = torch.Generator().manual_seed(0)
            prompt = lambda n: torch.randint(0, z["vocab"], (n,), generator=g).tolist()
            pre = min(engine.time_prefill(prompt(prefill_tokens), repeats=5))
            dt = engine.time_decode([prompt(context) for _ in range(batch)], steps=steps, warmup=warmup)
            row[label] = {"prefill_tok_s": round(prefill_tokens / pre, 1), "prefill_ms": round(pre * 1e3, 3),
                          "decode_tok_s": round(batch * steps / dt, 1), "decode_ms_per_step": round(dt / steps * 1e3, 4),
                          "weights_gb": round(engine.model.weight_bytes() / 1e9, 3)}
            print(f"[bench] {name} {label}: {row[label]}", file=sys.stderr, flush=True)
            del engine
            torch.cuda.empty_cache()
        row["kernels_prefill"] = _zudisun_kernels(z, prefill_tokens, context)
        row["kernels_decode"] = _zudisun_kernels(z, batch, context)
        print(f"[bench] {name} kernels: {row['kernels_prefill']} {row['kernels_decode']}", file=sys.stderr, flush=True)
        results[name] = row
    first = results[next(iter(results))]
    print(json.dumps({
        "metric": "Zudisun beside Gisodra and the dense Llama at equal sizes: prefill and decode tok/s", "unit": "tokens/s",
        "value": first["zudisun"]["decode_tok_s"], "n_gpus": 1, "steps": steps, "warmup": warmup, "higher_is_better": True,
        "dtype": "bf16", "data": "synthetic",
        "config": {"prefill_tokens": prefill_tokens, "decode_batch": batch, "decode_context": context, "page_size": PAGE,
                   "sizes": ZUDISUN_SIZES},
        "results": results,
    }), flush=True)
    return 0


# Sodotar at sizes that resemble a real model's layers: eight layers in the order differential attention, latent
# attention, differential attention on the first one's keys, latent attention, twice, each with a routed
# feed-forward and a gated shared expert, four residual streams.  A differential layer has half the heads of the
# models beside it, two maps a head and values twice as wide (as many score maps and as many value columns).
# Beside it: Gisodra (the framework's closest model: attention layers that read another layer's cache, latent
# attention) and the dense Llama, both of the same width, heads, head size and number of layers, whose dense
# feed-forward is as wide as the experts a token uses plus the shared one.
SODOTAR_SIZES = {
    "w1024": dict(width=1024, heads=16, kv_heads=4, dim=64, block=1024, lat_dim=64, rot_dim=32, kv_rank=192, streams=4,
                  experts=16, top=2, expert_ff=704, shared_ff=1408, vocab=32000),
    "w2048": dict(width=2048, heads=16, kv_heads=4, dim=128, block=4096, lat_dim=128, rot_dim=64, kv_rank=192, streams=4,
                  experts=32, top=4, expert_ff=768, shared_ff=2560, vocab=32000),
}


def _sodotar_configs(z: dict):
    mlp = dict(kind="moe", router=dict(experts=z["experts"], top=z["top"]), expert=dict(ff=z["expert_ff"], limit=7.0),
               shared=dict(ff=z["shared_ff"], limit=7.0))
    diff = lambda **more: dict(type="attention", mlp=mlp, mixer=dict(
        heads=z["heads"] // 2, kv_heads=z["kv_heads"] // 2, dim=z["dim"], vdim=2 * z["dim"], scale=z["dim"] ** -0.5, diff=0.8,
        mask=dict(size=z["block"]), rot=dict(base=500000.0, dims=z["dim"]), **more))
    latent = dict(type="latent_attention", mlp=mlp, mixer=dict(
        heads=z["heads"], dim=z["lat_dim"], rot_dim=z["rot_dim"], vdim=z["dim"], kv_rank=z["kv_rank"],
        scale=(z["lat_dim"] + z["rot_dim"]) ** -0.5, rot=dict(base=1000000.0, dims=z["rot_dim"])))
    layers = [diff(), latent, diff(kv_from=0), latent, diff(), latent, diff(kv_from=4), latent]
    new = dict(architecture="Sodotar", width=z["width"], vocab=z["vocab"], norm=dict(eps=1e-6), streams=z["streams"],
               logit_scale=0.5, layers=layers)
    ff = z["top"] * z["expert_ff"] + z["shared_ff"]
    g = dict(GISODRA_SIZES["w1024" if z["width"] == 1024 else "w2048"], ff=ff)
    hybrid, _ = _gisodra_configs(g)
    dense = dict(architectures=["LlamaForCausalLM"], hidden_size=z["width"], intermediate_size=ff,
                 num_hidden_layers=len(layers), num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"],
                 rms_norm_eps=1e-6, vocab_size=z["vocab"], rope_theta=500000.0, rope_scaling=None,
                 tie_word_embeddings=True, max_position_embeddings=131072)
    return new, hybrid, dense


def _sodotar_kernels(z: dict, rows: int, context: int) -> dict:
    """The design's own kernels at ``rows`` tokens (one prompt of ``rows`` tokens, or ``rows`` sequences of one
    token at ``context`` cached ones), each beside the like kernel of the closest model on operands of the same
    size: microseconds, and the shares of the memory roofline (the bytes the kernel has to move) and of the
    matrix cores' (its products' flops)."""
    import numpy as np
    import torch

    from fastgen_amd.kernels import ops

    D, H, G, d, P, S = z["width"], z["heads"], z["kv_heads"], z["dim"], PAGE, z["streams"]
    Hd, Gd, e = H // 2, G // 2, 2 * d  # the differential layer: heads, key/value heads, value width
    g = torch.Generator(device="cuda").manual_seed(rows)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device="cuda") * 0.05).to(torch.bfloat16)
    f32 = lambda *shape: torch.randn(*shape, generator=g, device="cuda")
    decode = rows <= 16
    out = {}

    def put(name, fn, nbytes, flops=0):
        t = _time(fn)
        out[name] = {"us": round(t * 1e6, 1), "hbm_frac": round(nbytes / t / PEAK_HBM, 4),
                     "mfma_frac": round(flops / t / PEAK_FLOPS["bf16"], 4)}

    # the streams' update, sum and norm; beside the one stream's addition and norm
    x, delta, w = f32(S, rows, D), rnd(rows, D), rnd(D)
    upd = ops.StreamUpdate(delta, f32(S, S), f32(S))
    normed = torch.empty(rows, D, dtype=torch.bfloat16, device="cuda")
    in_w = f32(S)
    put("streams_step", lambda: ops.streams_step(x, upd, in_w, w, 1e-6, normed), rows * D * (8 * S + 2 + 2))
    h = f32(rows, D)
    put("add_rmsnorm (one stream)", lambda: ops.add_rmsnorm(h, delta, w, 1e-6, normed), rows * D * (4 + 4 + 2 + 2))
    # between the q/k/v product and the attention: rotation, padding, cache write (the value goes in with both maps)
    n_seqs = rows if decode else 1
    keys = context + 1 if decode else rows
    pages_seq = -(-keys // P)
    n_pages = n_seqs * pages_seq
    hc = -(-max(d, e) // 16) * 16
    width = 2 * Hd * d + 2 * Gd * d + 2 * Gd * e
    src = f32(rows, width)
    kp, vp = rnd(n_pages, 2 * Gd, P, hc), rnd(n_pages, 2 * Gd, hc, P)
    table = ops.rope_table(torch.arange(rows, dtype=torch.int32, device="cuda"), f32(d // 2).abs())
    bt = torch.arange(n_pages, dtype=torch.int32, device="cuda").view(n_seqs, pages_seq)
    if decode:
        slots = (torch.arange(rows, dtype=torch.int32, device="cuda") * pages_seq * P + context).contiguous()
    else:
        slots = torch.arange(rows, dtype=torch.int32, device="cuda")
    q = torch.empty(rows, 2 * Hd * hc, dtype=torch.bfloat16, device="cuda")
    put("heads_prepare (two maps a head)", lambda: ops.heads_prepare(
        src, None, 1e-6, n_q=2 * Hd, q_col=0, q_width=d, q_out=q, q_out_width=hc, n_kv=2 * Gd, k_col=2 * Hd * d, k_width=d,
        v_col=2 * Hd * d + 2 * Gd * d, v_width=e, table=table, rot_start=0, rotary_dim=d, slots=slots, k_pages=kp, v_pages=vp),
        src.numel() * 4 + rows * (2 * Hd * hc + 4 * Gd * hc) * 2)
    src_g, nw = f32(rows, (H + 2 * G) * d), f32(d)
    kg, vg = rnd(n_pages, G, P, d), rnd(n_pages, G, d, P)
    qg = torch.empty(rows, H * d, dtype=torch.bfloat16, device="cuda")
    put("heads_prepare (gisodra attention)", lambda: ops.heads_prepare(
        src_g, None, 1e-6, n_q=H, q_col=0, q_width=d, q_norm=nw, q_norm_dims=d, q_out=qg, q_out_width=d, n_kv=G, k_col=H * d,
        k_width=d, k_norm=nw, k_norm_dims=d, v_col=(H + G) * d, v_width=d, slots=slots, k_pages=kg, v_pages=vg),
        src_g.numel() * 4 + rows * (H + 2 * G) * d * 2)
    # the attention itself: 2 Hd maps over 2 Gd key heads of the padded width and a mask of blocks, beside H heads
    # over G key heads of width d; the bytes are the keys and values that have to be read (a value once)
    if decode:
        q_lens, q_start, n_cached = [1] * rows, list(range(rows + 1)), [context] * rows
    else:
        q_lens, q_start, n_cached = [rows], [0, rows], [0]
    def attention(name, qq, k_pages, v_pages, heads, kv, window, need_bytes, flops):
        width = k_pages.shape[3]
        small, big = ops.attention_items(np.array(q_lens), np.array(q_start), np.array(n_cached), heads // kv,
                                         ops.attention_tile_rows(width, False, True))
        both = ops.upload(np.concatenate([small, big]).reshape(-1), torch.int32, "cuda")
        sm, bg = (both[: small.size] if small.size else None), (both[small.size:] if big.size else None)
        o = torch.empty(rows, heads * width, dtype=torch.bfloat16, device="cuda")
        put(name, lambda: ops.paged_attention_mfma(qq, o, k_pages, v_pages, bt, sm, bg, heads, 0.1, window, exact_weights=True),
            need_bytes, flops)
    seen = n_seqs * keys if decode else rows  # keys a sequence's tokens read (a prompt: each page once a tile row)
    pairs = n_seqs * keys if decode else rows * (rows + 1) // 2
    attention("attention (two maps a head, blocks)", q, kp, vp, 2 * Hd, 2 * Gd, ops.block_mask(z["block"]),
              seen * (2 * Gd * d + Gd * e) * 2, 2 * pairs * 2 * Hd * (d + e))
    attention("attention (gisodra: H heads)", qg, kg, vg, H, G, 0, seen * 2 * G * d * 2, 2 * pairs * H * 2 * d)
    att = rnd(rows, 2 * Hd * hc)
    o = torch.empty(rows, Hd * e, dtype=torch.bfloat16, device="cuda")
    put("head_diff_norm", lambda: ops.head_diff_norm(att, hc, o, Hd, Hd // Gd, e, 0.6, 1e-6, 0.2), rows * (2 * Hd * e + Hd * e) * 2)
    x32, gate16, nwe = f32(rows, H * d), rnd(rows, H * d), f32(d)
    og = torch.empty(rows, H * d, dtype=torch.bfloat16, device="cuda")
    put("head_norm_gate (gisodra)", lambda: ops.head_norm_gate(x32, nwe, 1e-6, gate16, H, og), rows * H * d * (4 + 2 + 2))
    # the router: softmax over all experts, correction, the shared expert's gate row; beside softmax over the chosen
    E, top, F = z["experts"], z["top"], z["expert_ff"]
    xr, router, corr = rnd(rows, D), f32(E + 1, D) * 0.05, f32(E) * 0.01
    put("moe_route (softmax over all, gate row)", lambda: ops.moe_route(xr, router, None, top, False, corr, 1, 1, 1.0, True, 1),
        router.numel() * 4 + rows * D * 2)
    r2 = router[:E].contiguous()
    put("moe_route (buderax)", lambda: ops.moe_route(xr, r2, None, top), r2.numel() * 4 + rows * D * 2)
    # the experts' first product with the limited activation, beside the same with SiLU
    choice, _ = ops.moe_route(xr, r2, None, top)
    tile_rows = 16 if decode else (128 if rows * top / E >= 96 else 64)
    sorted_, tiles = ops.moe_sort(choice, E, tile_rows)
    wg, wu = rnd(E, F, D), rnd(E, F, D)
    used = min(E, rows * top)
    put("moe_gate_up (limited)", lambda: ops.moe_gate_up(xr, wg, wu, sorted_, tiles, top, tile_rows, 7.0, 1.702),
        used * 2 * F * D * 2, 2 * rows * top * 2 * F * D)
    put("moe_gate_up (silu)", lambda: ops.moe_gate_up(xr, wg, wu, sorted_, tiles, top, tile_rows), used * 2 * F * D * 2,
        2 * rows * top * 2 * F * D)
    # the shared expert's activation on the product's fp32 rows, and the combine with its gate
    gu = f32(rows, 2 * z["shared_ff"])
    put("gated_mul (limited)", lambda: ops.gated_mul(gu, None, "limited", torch.bfloat16, None, 7.0, 1.702), rows * z["shared_ff"] * (8 + 2))
    gu16 = rnd(rows, 2 * z["shared_ff"])
    put("silu_mul (llama)", lambda: ops.silu_mul(gu16), rows * z["shared_ff"] * (4 + 2))
    y, wt, plus, pg = f32(rows * top, D), f32(rows, top), rnd(rows, D), f32(rows)
    put("moe_combine (gated shared expert)", lambda: ops.moe_combine(y, wt, plus, pg), rows * D * (4 * top + 2 + 4))
    put("moe_combine (buderax)", lambda: ops.moe_combine(y, wt, plus), rows * D * (4 * top + 2 + 4))
    return out


def sodotar_workload(prefill_tokens: int = 2048, batch: int = 8, context: int = 1024, steps: int = 32, warmup: int = 8) -> int:
    """Prefill and decode throughput of Sodotar models with random bfloat16 weights beside Gisodra and dense Llama
    models of equal sizes, and the design's own kernels beside the other models' like ones.  One JSON line."""
    import torch

    from fastgen_amd.engine import Engine

    results = {}
    for name, z in SODOTAR_SIZES.items():
        new, hybrid, dense = _sodotar_configs(z)
        row = {"layers": len(new["layers"])}
        for label, cfg in (("sodotar", new), ("gisodra", hybrid), ("llama", dense)):
            engine = Engine.from_config(cfg, seed=5, dtype=torch.bfloat16, page_size=PAGE,
                                        max_tokens=max(batch * (context + 256), prefill_tokens + PAGE), max_batch=batch,
                                        max_step_tokens=prefill_tokens)
            g = torch.Generator().manual_seed(0)
            prompt = lambda n: torch.randint(0, z["vocab"], (n,), generator=g).tolist()
            pre = min(engine.time_prefill(prompt(prefill_tokens), repeats=5))
            dt = engine.time_decode([prompt(context) for _ in range(batch)], steps=steps, warmup=warmup)
            row[label] = {"prefill_tok_s": round(prefill_tokens / pre, 1), "prefill_ms": round(pre * 1e3, 3),
                          "decode_tok_s": round(batch * steps / dt, 1), "decode_ms_per_step": round(dt / steps * 1e3, 4),
                          "weights_gb": round(engine.model.weight_bytes() / 1e9, 3)}
            print(f"[bench] {name} {label}: {row[label]}", file=sys.stderr, flush=True)
            del engine
            torch.cuda.empty_cache()
        row["kernels_prefill"] = _sodotar_kernels(z, prefill_tokens, context)
        row["kernels_decode"] = _sodotar_kernels(z, batch, context)
        print(f"[bench] {name} kernels: {row['kernels_prefill']} {row['kernels_decode']}", file=sys.stderr, flush=True)
        results[name] = row
    first = results[next(iter(results))]
    print(json.dumps({
        "metric": "Sodotar beside Gisodra and the dense Llama at equal sizes: prefill and decode tok/s", "unit": "tokens/s",
        "value": first["sodotar"]["decode_tok_s"], "n_gpus": 1, "steps": steps, "warmup": warmup, "higher_is_better": True,
        "dtype": "bf16", "data": "synthetic",
        "config": {"prefill_tokens": prefill_tokens, "decode_batch": batch, "decode_context": context, "page_size": PAGE,
                   "sizes": SODOTAR_SIZES},
        "results": results,
    }), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default=None,
                    help="layer sizes: Llama 3.1 8B (the benchmark's configuration; default but for serve), 70B"
                         " (141 GB of weights) or Llama 3.2 3B (the default of serve)")
    ap.add_argument("--prefill-tokens", type=int, default=PROMPT_LEN,
                    help="tokens of the timed prefill step (default: the benchmark's 2,048)")
    ap.add_argument("--context", type=int, default=None,
                    help="cached tokens of each request when the timed decode steps begin (default: the prompt's"
                         " 2,048); more are fed untimed, in portions")
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--workload", choices=["decode", "serve", "readme", "buderax", "gisodra", "zudisun", "sodotar"], default="decode",
                    help="decode (default): the step benchmark; serve: continuous batching of 256 requests; "
                         "readme: the load of the reference's README; buderax, gisodra, zudisun, sodotar: that design beside the "
                         "dense Llama at equal sizes")
    ap.add_argument("--step-budget", type=int, default=2048, help="tokens a step of the serve workload")
    ap.add_argument("--show-choices", action="store_true",
                    help="print (stderr) which kernel the run's measurements chose for each matrix product")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported", flush=True)
        return 2
    if a.workload == "serve":
        return serve_workload(step_budget=a.step_budget, shape=a.shape or "3b")
    if a.workload == "readme":
        return readme_workload(a.shape or "8b")
    if a.workload == "gisodra":
        return gisodra_workload(prefill_tokens=a.prefill_tokens, batch=a.batch, steps=min(a.steps, 32), warmup=a.warmup)
    if a.workload == "sodotar":
        return sodotar_workload(prefill_tokens=a.prefill_tokens, batch=a.batch, steps=min(a.steps, 32), warmup=a.warmup)
    if a.workload == "zudisun":
        return zudisun_workload(prefill_tokens=a.prefill_tokens, batch=a.batch, steps=min(a.steps, 32), warmup=a.warmup)
    if a.workload == "buderax":
        return buderax_workload(prefill_tokens=a.prefill_tokens, batch=a.batch, steps=min(a.steps, 32), warmup=a.warmup)
    a.shape = a.shape or "8b"

    import torch

    from fastgen_amd.engine import Engine

    dtype = {"bf16": torch.bfloat16, "fp32": torch.float32}[a.dtype]
    model_name, shape = SHAPES[a.shape]
    full_layers = shape["num_hidden_layers"]
    a.layers = a.layers or full_layers
    cfg = dict(shape, num_hidden_layers=a.layers)
    batches = sorted({a.batch} | (set() if a.no_points else {1, 64}))
    max_b = max(batches)
    t0 = time.time()
    # The cache holds CONTEXT_LEN tokens for every request of the largest batch (68.7 GB at batch 64 of the 8B
    # shape in bfloat16), or what the GPU has free beside the weights if that is less (the 70B shape); with
    # --context, as many as the requests reach: the first requests of a batch decode while the prompts of the
    # later ones are still fed in portions, so they are longer than --context by the number of those steps.
    from fastgen_amd.engine import Model

    ctx_len = a.context or PROMPT_LEN
    feed_steps = -(-max_b * ctx_len // max(1, PROMPT_LEN - max_b)) + max_b
    capacity = max(CONTEXT_LEN, -(-(ctx_len + feed_steps + a.warmup + a.steps + 72) // PAGE) * PAGE,
                   -(-a.prefill_tokens // PAGE) * PAGE)
    if capacity > cfg["max_position_embeddings"]:
        print(f"bench.py: --context {ctx_len} and the steps after it pass the model's {cfg['max_position_embeddings']}"
              " positions", flush=True)
        return 2
    model = Model.random(cfg, 2, dtype, "cuda:0")
    engine = Engine(model, page_size=PAGE, max_tokens=None, max_batch=max_b, max_step_tokens=PROMPT_LEN,
                    max_seq=capacity)
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    model = engine.model
    D, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    H, KV = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd, L = D // H, a.layers
    esize = 2 if a.dtype == "bf16" else 4
    layer_params = D * (H + 2 * KV) * hd + H * hd * D + 3 * D * F
    kv_bytes_per_token = 2 * KV * hd * esize * L

    g = torch.Generator().manual_seed(0)

    def prompt(n):
        return torch.randint(0, V, (n,), generator=g).tolist()

    # ------------------------------------------------------------ prefill
    times = engine.time_prefill(prompt(a.prefill_tokens), repeats=5)
    pre = sum(times) / len(times)  # the mean of the repeats after one warm-up; the best is reported beside it
    T = a.prefill_tokens
    flops = 2 * T * L * layer_params + L * 4 * H * hd * (T * (T + 1) // 2) + 2 * D * V
    prefill = {"value": round(T / pre, 1), "tokens": T, "ms": round(pre * 1e3, 3),
               "frac": round(flops / pre / PEAK_FLOPS[a.dtype], 4), "repeats": len(times),
               "best_ms": round(min(times) * 1e3, 3)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ------------------------------------------------------------- decode
    results = {}
    for b in batches:
        steps, warm = (a.steps, a.warmup)
        dt = engine.time_decode([prompt(ctx_len) for _ in range(b)], steps=steps, warmup=warm)
        ctx = engine.last_mean_context  # mean cached tokens of a request during the timed steps
        nbytes = (L * layer_params + D * V) * esize + b * ctx * kv_bytes_per_token
        results[b] = dict(tok_s=b * steps / dt, ms=dt / steps * 1e3, gbs=nbytes / (dt / steps) / 1e9, ctx=ctx)
        print(f"[bench] decode batch {b}: {results[b]}", file=sys.stderr, flush=True)

    r = results[a.batch]
    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2048 tokens; % of roofline",
        "value": round(r["tok_s"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(r["ms"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic",
        "config": {
            "model": model_name, "global_batch": a.batch, "seq_len": capacity, "mean_context": round(r["ctx"], 1),
            "prompt_len": ctx_len, "cache_tokens": engine.scheduler.pool_tokens, "parallelism": "none", "layers": L, "layers_full": full_layers,
            "hidden": D, "heads": H, "kv_heads": KV, "head_dim": hd, "ffn": F, "vocab": V, "page_size": PAGE,
            "rope_theta": cfg["rope_theta"], "rope_factor": cfg["rope_scaling"]["factor"], "norm_eps": cfg["rms_norm_eps"],
            # 2: every matrix is also held in the order the decode products read it (the roofline's bytes count one)
            "weight_copies": 2 if model.packed() else 1,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(r["gbs"], 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(r["gbs"] * 1e9 / PEAK_HBM, 4)},
        "points": {f"decode_b{b}": round(v["tok_s"], 1) for b, v in results.items() if b != a.batch},
    }
    print(json.dumps(line), flush=True)
    if a.show_choices:
        from fastgen_amd.kernels import linear

        for (what, n, k, rows), name in sorted(linear.choices.items(), key=lambda kv: (kv[0][1], kv[0][2], kv[0][0], kv[0][3])):
            took = ", ".join(f"{c} {1e3 * t:.1f} us" for c, t in sorted(linear.timings.get((what, n, k, rows), {}).items()))
            print(f"[bench] product {what} N={n} K={k} rows<={rows}: {name} ({took})", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
