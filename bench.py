#!/usr/bin/python3
"""Decode and prefill throughput of the MiniCPM-2B-shaped model on one MI355X.

  python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole batch: the scheduler's step (plan, the step
function over one new token per request, greedy sampling on the device, the sampled
tokens fed back and the finish rules checked); the reference times the same loop,
scripts/jiuge.py:562-583, prefill excluded.  Weights are random (seeded), prompts are
seeded uniform-random token ids.  One JSON line is printed.

  --workload mixed   the 1B shape's workload: 64 requests, prompts of 128..2,048 tokens, portions of 512
  --workload long    the 8B shape's workload: 4 prompts of 16,384 tokens, then decoding
  --direct           decode by calling the step function directly, without the scheduler
  --workload designs the Fopezen, Mezinex, Daborax and Fizelix decoders beside the MiniCPM decoder at equal layer sizes
                     (a few layers of three real models' sizes): prefill and decode throughput of each, with the fraction
                     of the memory or matrix-core peak it reaches (--only <design>: one of them, for a profiler)
"""
import argparse
import json
import math
import os
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

# The benchmark's configuration: MiniCPM-2B-shaped (40 layers, hidden 2304, 36 heads of 64, vocabulary 122753)
MODEL = dict(
    model_type="minicpm", vocab_size=122753, hidden_size=2304, num_hidden_layers=40,
    num_attention_heads=36, num_key_value_heads=36, intermediate_size=5760,
    max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=10000.0,
    scale_emb=12, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=True, eos_token_id=2)
# Two further shapes for --shape: MiniCPM-1B-shaped (deep, narrow, 3 query heads per kv head) and
# MiniCPM4-8B/FM9G-8B-shaped (16 query heads per kv head, head size 128, longrope).  The default run is 2b.
def _seeded_factors(seed, n=64):
    """Long-context rotary factors drawn from the seed, uniform in [1, 4]."""
    import random
    rng = random.Random(seed)
    return [1.0 + 3.0 * rng.random() for _ in range(n)]


SHAPES = {
    "2b": MODEL,
    "1b": dict(MODEL, vocab_size=73440, hidden_size=1536, num_hidden_layers=52, num_attention_heads=24,
               num_key_value_heads=8, intermediate_size=3840),
    "8b": dict(MODEL, vocab_size=73448, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
               num_key_value_heads=2, intermediate_size=16384, rms_norm_eps=1e-6, tie_word_embeddings=False,
               max_position_embeddings=32768,
               rope_scaling=dict(type="longrope", original_max_position_embeddings=32768,
                                 short_factor=_seeded_factors(1), long_factor=_seeded_factors(2))),
}
PROMPT = 2048
BATCH = 8
WEIGHT_STD = 0.1


def _sync():
    torch.cuda.synchronize()


DTYPE = torch.bfloat16          # --dtype float32: the whole model in true 32-bit (weights, activations, cache, products)


def _elem_bytes():
    return 2 if DTYPE == torch.bfloat16 else 4


def build_engine(layers, max_tokens, max_requests, page_size):
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights
    cfg = dict(MODEL, num_hidden_layers=layers or MODEL["num_hidden_layers"])
    conf = config_from_dict(cfg)
    model = build_model(conf.model_spec(), Runtime(dtype=DTYPE, device="cuda:0"))
    init_random_weights(model, seed=0, std=WEIGHT_STD, tie=bool(cfg.get("tie_word_embeddings", True)))
    return Engine(model, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests), conf


def model_numbers(conf):
    """Bytes of weights a decode step reads once, cache bytes per token, flops per prefill."""
    d, L, di, V = conf.hidden_size, conf.num_hidden_layers, conf.intermediate_size, conf.vocab_size
    nh, nkvh, dh = conf.num_attention_heads, conf.num_key_value_heads, conf.head_dim
    per_layer = (nh + 2 * nkvh) * dh * d + nh * dh * d + 3 * d * di
    eb = _elem_bytes()
    weight_bytes = eb * (L * per_layer + V * d) + 4 * d * (2 * L + 1)      # the head's table once; embedding rows are negligible
    kv_bytes_per_token = 2 * L * nkvh * dh * eb

    def prefill_flops(T):
        linear = 2.0 * T * L * per_layer
        attn = L * nh * dh * 4.0 * (T * (T + 1) / 2)        # QK^T and PV over the causal half
        head = 2.0 * V * d                                   # last row only
        return linear + attn + head
    return weight_bytes, kv_bytes_per_token, prefill_flops


def time_prefill(engine, tokens, reps=6):
    """Mean time of a whole-prompt step with its sampled token (one untimed pass first)."""
    from infinicore_infer_amd.engine import StepEntry
    total = 0.0
    for i in range(reps + 1):
        _sync()
        t0 = time.perf_counter()
        logits = engine.step([StepEntry("pf", tokens, [len(tokens) - 1])])
        engine.sample(logits)
        _sync()
        dt = time.perf_counter() - t0
        engine.free("pf")
        if i > 0:
            total += dt
    return total / reps


def time_decode_scheduled(engine, batch, steps, warmup, vocab, seed=0):
    """``batch`` requests of PROMPT tokens go through the scheduler; once all of them decode, ``warmup``
    untimed and ``steps`` timed steps (each: one token for every request)."""
    from infinicore_infer_amd.engine.scheduler import Scheduler
    from infinicore_infer_amd.engine.tasks import InferTask
    g = torch.Generator().manual_seed(seed)
    sch = Scheduler(engine, max_batch_tokens=max(PROMPT, batch), chunk_size=PROMPT, overlap=True)
    for i in range(batch):
        toks = torch.randint(0, vocab, (PROMPT,), generator=g).tolist()
        sch.add(InferTask("d%d" % i, toks, 1 << 30, temperature=0.0, topk=1, end_tokens=[],
                          max_new_tokens=warmup + steps + batch + 8))     # the first ones decode while the others' prompts run
    while sch.waiting or any(not r.decoding for r in sch.running):
        sch.step()
    # (decoding runs one step ahead of the host: a call issues at most one step and returns the tokens of the one before)
    first = sch.n_steps
    while sch.n_steps < first + warmup:
        sch.step()
    _sync()
    ctx0 = engine.length("d0")
    first = sch.n_steps
    t0 = time.perf_counter()
    while sch.n_steps < first + steps:
        sch.step()
    _sync()
    dt = time.perf_counter() - t0
    ctx1 = engine.length("d0")
    assert sch.n_steps == first + steps and ctx1 - ctx0 == steps
    assert len(sch.running) == batch and sch.n_preempted == 0
    for i in range(batch):
        sch.abort("d%d" % i)
    return dt / steps, (ctx0 + ctx1) / 2.0


def time_decode(engine, batch, steps, warmup, vocab, seed=0):
    """Prefill ``batch`` requests of PROMPT tokens, then time ``steps`` decode steps."""
    from infinicore_infer_amd.engine import StepEntry
    g = torch.Generator().manual_seed(seed)
    ids = ["d%d" % i for i in range(batch)]
    last = []
    for rid in ids:
        toks = torch.randint(0, vocab, (PROMPT,), generator=g).tolist()
        logits = engine.step([StepEntry(rid, toks, [PROMPT - 1])])
        last.append(engine.sample(logits)[0])

    def one():
        nonlocal last
        logits = engine.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, last)])
        last = engine.sample(logits)

    for _ in range(warmup):
        one()
    _sync()
    ctx0 = engine.length(ids[0])
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    _sync()
    dt = time.perf_counter() - t0
    ctx1 = engine.length(ids[0])
    for rid in ids:
        engine.free(rid)
    return dt / steps, (ctx0 + ctx1) / 2.0


# Layer sizes for --workload designs: (width, heads, kv heads, head size, feed-forward, vocabulary).  The Fopezen model has the
# same width, heads, kv heads and key size; its value size, window and kept keys are listed beside.
DESIGN_SIZES = {
    "2b-like": dict(width=2304, heads=36, kv=36, dim=64, ff=5760, vocab=32000, vdim=64, window=1024, keep=4),
    "8b-like": dict(width=4096, heads=32, kv=8, dim=128, ff=14336, vocab=32000, vdim=128, window=2048, keep=16),
    "1b-like": dict(width=1536, heads=24, kv=8, dim=64, ff=3840, vocab=32000, vdim=32, window=512, keep=4),
}


def _design_configs(z, layers):
    mini = dict(model_type="minicpm", vocab_size=z["vocab"], hidden_size=z["width"], num_hidden_layers=layers,
                num_attention_heads=z["heads"], num_key_value_heads=z["kv"], head_dim=z["dim"], intermediate_size=z["ff"],
                max_position_embeddings=8192, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True, eos_token_id=[])
    mixer = lambda w, k: dict(heads=z["heads"], kv_heads=z["kv"], dim=z["dim"], vdim=z["vdim"], scale=z["dim"] ** -0.5,
                              mask=dict(size=w, keep_first=k), v_mix=True)
    kinds = ["attention", "attention", "attention_2", "attention"]
    fop = dict(architecture="Fopezen", vocab=z["vocab"], width=z["width"], norm=dict(eps=1e-5),
               layers=[dict(type=kinds[i % 4], mixer=mixer(z["window"], z["keep"]), mlp=dict(kind="dense", ff=z["ff"]))
                       for i in range(layers)])
    # Mezinex at the same width and feed-forward: latent attention with the same heads and plain key size (a rotated part of
    # 64 or 32, a latent of 512 or 256, a query latent of a third of the width), a gated linear recurrence as wide as the
    # model with one gate block per head, a state-space mixer of twice the width in heads of 64 with states of 128; two
    # residual streams and a pair table
    big = z["dim"] >= 128
    latent = dict(heads=z["heads"], dim=z["dim"], rot_dim=64 if big else 32, vdim=z["dim"], q_rank=z["width"] // 3 // 64 * 64,
                  kv_rank=512 if big else 256, scale=(z["dim"] + (64 if big else 32)) ** -0.5,
                  rot=dict(base=1000000.0, dims=64 if big else 32))
    rglru = dict(width=z["width"], blocks=z["heads"], conv=4)
    ssm = dict(heads=2 * z["width"] // 64, vdim=64, state=128, groups=8, norm_groups=8, conv=4)
    mez_kinds = [("latent_attention", latent), ("rglru", rglru), ("mamba2", ssm), ("latent_attention", latent)]
    mez = dict(architecture="Mezinex", vocab=z["vocab"], width=z["width"], norm=dict(eps=1e-5), logit_scale=1.0, streams=2,
               embedding=dict(bigram=dict(buckets=65521, mul_prev=127, mul_cur=17)),
               layers=[dict(type=mez_kinds[i % 4][0], mixer=mez_kinds[i % 4][1], mlp=dict(kind="dense", ff=z["ff"]))
                       for i in range(layers)])
    # Daborax at the same width and feed-forward: attention with the same heads, kv heads, key and value sizes and window as
    # Fopezen's (a cap on the scores, learned sinks, no kept keys), linear attention with a decay per head in heads of the
    # same size, and the state-space mixer of the Mezinex configuration; the fourth layer runs with the first one's tensors
    dab_att = dict(heads=z["heads"], kv_heads=z["kv"], dim=z["dim"], vdim=z["vdim"], scale=z["dim"] ** -0.5, softcap=50.0,
                   mask=dict(size=z["window"]))
    dab_lin = dict(heads=z["heads"], dim=z["dim"], vdim=z["dim"], decay=[1.0 - 2.0 ** (-5 - 3 * h / z["heads"]) for h in range(z["heads"])])
    dab_kinds = [("attention", dab_att), ("lightning", dab_lin), ("mamba2", ssm)]
    dab_layers = []
    for i in range(layers):
        l = dict(type=dab_kinds[i % 4 % 3][0], mixer=dab_kinds[i % 4 % 3][1], mlp=dict(kind="dense", ff=z["ff"], limit=7.0))
        if i % 4 == 3:
            l["weights_of"] = i - 3
        dab_layers.append(l)
    dab = dict(architecture="Daborax", vocab=z["vocab"], width=z["width"], norm=dict(eps=1e-5), embedding=dict(scale=1.0),
               residual_mult=0.5, layers=dab_layers)
    # Fizelix at the same width: attention with the same heads, kv heads, key and value sizes and window as Fopezen's (half of
    # every head rotated, one mean key and value per block of 64 tokens before the window, sigmoid weights), the state-space
    # mixer of the Mezinex configuration; the feed-forwards are dense (the row's size) in the first and last layer and in
    # between eight experts of a quarter of that size, two per token, beside a shared one of the same size; a gate on every
    # sublayer's result and a token input of 64 columns per layer
    fiz_att = dict(heads=z["heads"], kv_heads=z["kv"], dim=z["dim"], vdim=z["vdim"], scale=z["dim"] ** -0.5,
                   mask=dict(size=z["window"], pool=64), rot=dict(base=500000.0, dims=z["dim"] // 2))
    fiz_moe = dict(kind="moe", router=dict(experts=8, top=2), expert=dict(ff=z["ff"] // 4), shared=dict(ff=z["ff"] // 4))
    fiz_kinds = [("attention", fiz_att, dict(kind="dense", ff=z["ff"])), ("mamba2", ssm, fiz_moe), ("attention", fiz_att, fiz_moe),
                 ("mamba2", ssm, dict(kind="dense", ff=z["ff"]))]
    fiz = dict(architecture="Fizelix", vocab=z["vocab"], width=z["width"], norm=dict(eps=1e-5), embedding=dict(scale=1.0),
               logit_scale=1.0, token_side=dict(dim=64),
               layers=[dict(type=fiz_kinds[i % 4][0], mixer=fiz_kinds[i % 4][1], mlp=fiz_kinds[i % 4][2]) for i in range(layers)])
    return {"minicpm": mini, "fopezen": fop, "mezinex": mez, "daborax": dab, "fizelix": fiz}


def _design_numbers(design, z, layers, kinds=None):
    """(weight bytes a decode step reads, cache bytes a decode step reads per request at context n, prefill flops at T)."""
    d, H, G, dk, ff, V = z["width"], z["heads"], z["kv"], z["dim"], z["ff"], z["vocab"]
    eb = _elem_bytes()
    if design == "mezinex":
        return _mezinex_numbers(z, layers)
    if design == "daborax":
        return _daborax_numbers(z, layers)
    if design == "fizelix":
        return _fizelix_numbers(z, layers)
    if design == "minicpm":
        per_layer = (H + 2 * G) * dk * d + H * dk * d + 3 * d * ff
        kv = lambda n: 2 * layers * G * dk * eb * n
        attn = lambda T: layers * H * dk * 4.0 * (T * (T + 1) / 2)
    else:
        dv, w, keep = z["vdim"], z["window"], z["keep"]
        gated = sum(1 for i in range(layers) if i % 4 != 2)
        per_layer = (H * dk + G * dk + G * dv) * d + H * dv * d + 2 * d * ff
        per_layer += gated / layers * H * dv * d
        seen = lambda n: min(n, w + keep)
        kv = lambda n: layers * G * (dk + dv) * eb * seen(n)
        attn = lambda T: layers * H * (dk + dv) * 2.0 * sum(seen(i + 1) for i in range(T))
    weights = eb * (layers * per_layer + V * d)
    return weights, kv, (lambda T: 2.0 * T * layers * per_layer + attn(T) + 2.0 * V * d)


def _mezinex_numbers(z, layers):
    """As ``_design_numbers`` for the Mezinex configuration of ``_design_configs``: weights a decode step reads, bytes of
    cache and state it reads per request, flops of a prompt (products, the walk over the latent rows, the recurrences)."""
    cfg = _design_configs(z, layers)["mezinex"]
    d, ff, V, eb = z["width"], z["ff"], z["vocab"], _elem_bytes()
    weights, per_tok_lin, cache_row, state_bytes = V * d, 0.0, 0.0, 0.0
    walk = []          # (heads, row width + latent width) per attention layer: flops of the walk per (query, key) pair / 2
    scan = 0.0         # flops per token of the recurrences
    for l in cfg["layers"]:
        m = l["mixer"]
        n = 3 * d * ff
        if l["type"] == "latent_attention":
            H, R, E = m["heads"], m["kv_rank"], m["rot_dim"]
            n += (m["q_rank"] + R + E + H * m["vdim"]) * d + H * (m["dim"] + E) * m["q_rank"] + H * m["dim"] * R + H * m["vdim"] * R + d * H * m["vdim"]
            cache_row += (R + E) * eb
            walk.append(H * (2 * R + E))
        elif l["type"] == "rglru":
            w = m["width"]
            n += 3 * w * d + 2 * w * (w // m["blocks"])
            state_bytes += 2 * 4 * w * m["conv"]
            scan += 12.0 * w
        else:
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            n += (2 * inner + 2 * gn + m["heads"]) * d + d * inner
            state_bytes += 2 * 4 * (inner * m["state"] + (m["conv"] - 1) * (inner + 2 * gn))
            scan += 6.0 * inner * m["state"]
        weights += n
        per_tok_lin += 2.0 * n
    kv = lambda n: cache_row * n + state_bytes
    flops = lambda T: T * (per_tok_lin + scan) + sum(2.0 * w for w in walk) * (T * (T + 1) / 2) + 2.0 * V * d
    return eb * weights, kv, flops


def _daborax_numbers(z, layers):
    """As ``_design_numbers`` for the Daborax configuration of ``_design_configs``.  A layer that runs with another's tensors
    reads them again (they are counted per run: at these sizes a layer's matrices do not stay in the caches)."""
    cfg = _design_configs(z, layers)["daborax"]
    d, V, eb = z["width"], z["vocab"], _elem_bytes()
    weights, per_tok_lin, scan, state_bytes = V * d, 0.0, 0.0, 0.0
    spans = []         # (heads * (key + value size), kv heads * (key + value size), window) per attention layer
    for l in cfg["layers"]:
        m = l["mixer"]
        n = 3 * d * l["mlp"]["ff"]
        if l["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            n += (H * dk + G * dk + G * dv) * d + d * H * dv
            spans.append((H * (dk + dv), G * (dk + dv), m["mask"]["size"]))
        elif l["type"] == "lightning":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            n += (2 * H * dk + 2 * H * dv) * d + d * H * dv
            state_bytes += 2 * 4 * H * dk * dv
            scan += 6.0 * H * dk * dv
        else:
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            n += (2 * inner + 2 * gn + m["heads"]) * d + d * inner
            state_bytes += 2 * 4 * (inner * m["state"] + (m["conv"] - 1) * (inner + 2 * gn))
            scan += 6.0 * inner * m["state"]
        weights += n
        per_tok_lin += 2.0 * n
    kv = lambda n: sum(g * eb * min(n, w) for _, g, w in spans) + state_bytes
    flops = lambda T: T * (per_tok_lin + scan) + sum(2.0 * h * sum(min(i + 1, w) for i in range(T)) for h, _, w in spans) + 2.0 * V * d
    return eb * weights, kv, flops


def _fizelix_numbers(z, layers):
    """As ``_design_numbers`` for the Fizelix configuration of ``_design_configs``.  The weights a decode step reads depend
    on the batch: of a routed feed-forward's experts it reads those that some token chose, E (1 - (1 - top/E)^batch) on
    average, so the first number is a function of the batch."""
    cfg = _design_configs(z, layers)["fizelix"]
    d, V, eb = z["width"], z["vocab"], _elem_bytes()
    side = cfg["token_side"]["dim"]
    fixed, per_tok_lin, scan, state_bytes = V * d, 0.0, 0.0, 0.0
    routed = []        # (experts, top, weights of one expert) per routed feed-forward
    spans = []         # (heads * (key + value size), kv heads * (key + value size), window, block) per attention layer
    for l in cfg["layers"]:
        m, mlp = l["mixer"], l["mlp"]
        n = 2 * d * d + 2 * side * d                     # the two gates on the sublayers' results, the token input
        if l["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            n += (H * dk + G * dk + G * dv) * d + d * H * dv
            spans.append((H * (dk + dv), G * (dk + dv), m["mask"]["size"], m["mask"]["pool"]))
        else:
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            n += (2 * inner + 2 * gn + m["heads"]) * d + d * inner
            state_bytes += 2 * 4 * (inner * m["state"] + (m["conv"] - 1) * (inner + 2 * gn))
            scan += 6.0 * inner * m["state"]
        active = n
        if mlp["kind"] == "dense":
            n += 3 * d * mlp["ff"]
            active = n
        else:
            E, top, one = mlp["router"]["experts"], mlp["router"]["top"], 3 * d * mlp["expert"]["ff"]
            n += E * d + 3 * d * mlp["shared"]["ff"]
            active = n + top * one
            routed.append((E, top, one))
        fixed += n
        per_tok_lin += 2.0 * active
    seen = lambda n, w, p: min(n, w) + max(0, n - w) // p
    weights = lambda batch: eb * (fixed + sum(E * (1.0 - (1.0 - top / E) ** batch) * one for E, top, one in routed))
    kv = lambda n: sum(g * eb * seen(n, w, p) for _, g, w, p in spans) + state_bytes
    flops = lambda T: (T * (per_tok_lin + scan) + sum(2.0 * h * sum(seen(i + 1, w, p) for i in range(T)) for h, _, w, p in spans)
                       + 2.0 * V * d)
    return weights, kv, flops


def run_designs(args):
    """Prefill and decode of the two decoders at equal layer sizes.  Decoding calls the step function directly (recorded
    steps), greedy sampling on the device; a row gives tokens/s and what fraction of the memory bandwidth (decoding:
    weights once + the cache rows a step reads) or of the matrix-core peak (prefill) that is."""
    global PROMPT
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights
    PROMPT = args.prompt
    layers = args.layers or 4
    dname = "bf16" if DTYPE == torch.bfloat16 else "fp32"
    batches = [args.batch] if args.no_points else [1, 8, 64]
    rows = []
    for size in (args.sizes.split(",") if args.sizes else list(DESIGN_SIZES)):
        z = DESIGN_SIZES[size]
        for design, cfg in _design_configs(z, layers).items():
            if args.only and design != args.only:
                continue
            conf = config_from_dict(cfg)
            model = build_model(conf.model_spec(), Runtime(dtype=DTYPE, device="cuda:0"))
            init_random_weights(model, seed=0, std=0.02, norm_std=0.02)
            per_req = (PROMPT + args.warmup + args.steps + 128 + 63) // 64 * 64
            engine = Engine(model, max_tokens=per_req * max(batches), page_size=args.page_size, max_requests=max(batches) + 1)
            if args.eager:
                engine.use_graphs = False
            if not args.no_tune:
                engine.tune_library_products([PROMPT] + [b for b in batches if b > 16])
            weights, kv, pf_flops = _design_numbers(design, z, layers)
            g = torch.Generator().manual_seed(5)
            t_pf = time_prefill(engine, torch.randint(0, z["vocab"], (PROMPT,), generator=g).tolist(), reps=4)
            row = {"size": size, "design": design, "layers": layers,
                   "prefill_tokens_per_s": round(PROMPT / t_pf, 1), "prefill_ms": round(t_pf * 1e3, 3),
                   "prefill_frac_of_matrix_peak": round(pf_flops(PROMPT) / t_pf / (PEAK_TFLOPS[dname] * 1e12), 4), "decode": {}}
            for b in batches:
                dt, ctx = time_decode(engine, b, args.steps, args.warmup, z["vocab"], seed=b)
                row["decode"]["batch %d" % b] = {"tokens_per_s": round(b / dt, 1), "ms_per_step": round(dt * 1e3, 4),
                                                 "frac_of_hbm_peak": round(((weights(b) if callable(weights) else weights) + b * kv(ctx)) / dt / 1e9 / HBM_PEAK_GBS, 4)}
            rows.append(row)
            print(json.dumps(row), file=sys.stderr, flush=True)
            del engine, model
            torch.cuda.empty_cache()
    print(json.dumps({"metric": "prefill and decode tokens/s of the decoder designs at equal layer sizes", "unit": "tokens/s",
                      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": dname, "prompt": PROMPT,
                      "data": "synthetic (seeded random weights and token ids)", "rows": rows}))
    return 0


def run_mixed(args):
    """The 1B-shaped configuration's workload: 64 requests with prompts of 128..2,048 tokens go through the
    scheduler, which cuts the prompts into portions of 512 under a token budget per step and decodes the
    running requests beside them.  One JSON line: all tokens (prompt and generated) per second."""
    import random
    from infinicore_infer_amd.engine.scheduler import Scheduler
    from infinicore_infer_amd.engine.tasks import InferTask
    n_req, gen, chunk, budget = args.requests, args.steps, 512, args.token_budget
    rnd = random.Random(0)
    lens = [rnd.randint(128, 2048) for _ in range(n_req)]
    pool = sum((l + gen + args.page_size - 1) // args.page_size * args.page_size for l in lens) + 64 * args.page_size
    engine, conf = build_engine(args.layers, pool, n_req, args.page_size)
    if not args.no_tune:
        # the two step sizes that recur: a full token budget, and one token of every request
        engine.tune_library_products([budget] + [b for b in (n_req,) if b > 16])
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, conf.vocab_size, (l,), generator=g).tolist() for l in lens]

    def run():
        sch = Scheduler(engine, max_batch_tokens=budget, chunk_size=chunk, overlap=True)
        for i, toks in enumerate(prompts):
            sch.add(InferTask(i, toks, conf.max_position_embeddings, temperature=0.0, topk=1, end_tokens=[], max_new_tokens=gen))
        _sync()
        t0 = time.perf_counter()
        steps = []
        while sch.has_unfinished():
            s0, issued = time.perf_counter(), sch.n_steps
            sch.step()
            took = time.perf_counter() - s0
            if sch.n_steps > issued:                    # the call issued a step (while decoding runs ahead it also waited for the one before)
                steps.append((took, sum(n for _, _, n in sch.last_plan)))
            elif steps:                                 # it only read the tokens of the step in flight
                steps[-1] = (steps[-1][0] + took, steps[-1][1])
        _sync()
        return time.perf_counter() - t0, steps, sch.n_preempted

    run()                                            # one untimed pass: buffers grow, graphs are recorded
    dt, steps, preempted = run()
    total = sum(lens) + n_req * gen
    mixed = [s for s in steps if s[1] > n_req]
    dec = [s for s in steps if s[1] <= n_req]
    out = {
        "metric": "tokens/s (prompt + generated) through the scheduler, %d requests, prompts 128..2048, portions of %d "
                  "(MiniCPM-%s-shaped)" % (n_req, chunk, args.shape.upper()),
        "value": round(total / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": len(steps), "warmup": 1,
        "ms_per_step": round(dt / len(steps) * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (seeded random weights N(0,0.1) and token ids)",
        "config": {
            "model": "MiniCPM-%s-shaped" % args.shape.upper(), "layers": conf.num_hidden_layers, "layers_of_config": MODEL["num_hidden_layers"],
            "hidden": conf.hidden_size, "heads": conf.num_attention_heads, "kv_heads": conf.num_key_value_heads,
            "head_dim": conf.head_dim, "intermediate": conf.intermediate_size, "vocab": conf.vocab_size,
            "requests": n_req, "prompt_tokens": sum(lens), "generated_each": gen, "token_budget": budget, "portion": chunk,
            "page_size": args.page_size, "parallelism": "single-gpu", "sampling": "greedy on device",
        },
        "mixed_steps": {"count": len(mixed), "mean_ms": round(1e3 * sum(s[0] for s in mixed) / max(1, len(mixed)), 3),
                        "mean_tokens": round(sum(s[1] for s in mixed) / max(1, len(mixed)), 1)},
        "decode_steps": {"count": len(dec), "mean_ms": round(1e3 * sum(s[0] for s in dec) / max(1, len(dec)), 3)},
        "preempted": preempted,
    }
    weight_bytes, kv_per_tok, prefill_flops = model_numbers(conf)
    if mixed:      # a mixed step's matrix-product flops (its prompt portions dominate) against the bf16 peak
        d, L, di = conf.hidden_size, conf.num_hidden_layers, conf.intermediate_size
        per_tok = 2.0 * L * ((conf.num_attention_heads + 2 * conf.num_key_value_heads) * conf.head_dim * d
                             + conf.num_attention_heads * conf.head_dim * d + 3 * d * di)
        t_mixed = sum(s[0] for s in mixed) / len(mixed)
        n_mixed = sum(s[1] for s in mixed) / len(mixed)
        out["prefill"] = {"value": round(n_mixed / t_mixed, 1), "tokens": round(n_mixed, 1), "ms": round(t_mixed * 1e3, 3),
                          "frac": round(per_tok * n_mixed / t_mixed / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    if dec:        # a decode-only step reads every weight once and the live requests' cache
        t_dec = sum(s[0] for s in dec) / len(dec)
        ctx_mean = sum(lens) / len(lens) + gen / 2.0
        achieved = (weight_bytes + n_req * ctx_mean * kv_per_tok) / t_dec / 1e9
        out["roofline"] = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(achieved / HBM_PEAK_GBS, 4)}
    print(json.dumps(out))
    return 0


def main():
    global BATCH, MODEL, PROMPT, DTYPE
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--shape", default=None, choices=sorted(SHAPES), help="2b is the benchmark's configuration (default; 1b for --workload mixed)")
    ap.add_argument("--sizes", default=None, help="--workload designs: comma-separated sizes (default: all of 2b-like, 8b-like, 1b-like)")
    ap.add_argument("--only", default=None, choices=["fopezen", "minicpm", "mezinex", "daborax", "fizelix"], help="--workload designs: one design only")
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed", "long", "designs"],
                    help="decode: the benchmark (prefill of one prompt, decode steps at fixed batches); "
                         "mixed: 64 requests of 128..2048 prompt tokens through the scheduler, --steps tokens generated each; "
                         "long: the 8B shape with 4 prompts of 16,384 tokens (the same as --shape 8b --prompt 16384 --batch 4 --no-points)")
    ap.add_argument("--direct", action="store_true", help="decode through the step function directly, not through the scheduler")
    ap.add_argument("--requests", type=int, default=64, help="--workload mixed: number of requests")
    ap.add_argument("--token-budget", type=int, default=1024, help="--workload mixed: tokens per step")
    ap.add_argument("--prompt", type=int, default=PROMPT)
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--no-tune", action="store_true", help="keep the library's default kernel choice for prefill products")
    ap.add_argument("--batch", type=int, default=BATCH, help="batch of the headline run (for profiling other points)")
    ap.add_argument("--eager", action="store_true", help="decode without HIP graphs (so that a profiler's counters attribute to kernels)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"],
                    help="float32: the whole model in true 32-bit (no reduced-precision matrix mode), against the fp32 peak")
    args = ap.parse_args()
    DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    dname = "bf16" if DTYPE == torch.bfloat16 else "fp32"
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    if args.workload == "designs":
        if args.steps == ap.get_default("steps"):
            args.steps = 64
        return run_designs(args)
    if args.workload == "long":
        args.shape = args.shape or "8b"
        if args.prompt == ap.get_default("prompt"):
            args.prompt = 16384
        if args.batch == ap.get_default("batch"):
            args.batch = 4
        args.no_points = True
    if args.shape is None:
        args.shape = "1b" if args.workload == "mixed" else "2b"
    MODEL, PROMPT = SHAPES[args.shape], args.prompt
    if args.workload == "mixed":
        if args.steps == ap.get_default("steps"):
            args.steps = 64
        return run_mixed(args)
    per_req = PROMPT + args.warmup + args.steps + 64 + max(BATCH, args.batch, 64)
    per_req = (per_req + 63) // 64 * 64
    BATCH = args.batch
    batches = [BATCH] if args.no_points else sorted({BATCH, 1, 64}, key=lambda b: (b != BATCH, b))
    engine, conf = build_engine(args.layers, per_req * max(batches), max(batches) + 1, args.page_size)
    weight_bytes, kv_per_tok, prefill_flops = model_numbers(conf)
    vocab = conf.vocab_size
    if args.eager:
        engine.use_graphs = False

    if not args.no_tune:
        # the library's algorithm choice for the products of the prefill and of decoding at batches beyond 16
        engine.tune_library_products([PROMPT] + [b for b in batches if b > 16])
    g = torch.Generator().manual_seed(123)
    ptoks = torch.randint(0, vocab, (PROMPT,), generator=g).tolist()
    t_pf = time_prefill(engine, ptoks)
    pf_flops = prefill_flops(PROMPT)

    results = {}
    decode = time_decode if args.direct else time_decode_scheduled
    for b in batches:
        results[b] = decode(engine, b, args.steps, args.warmup, vocab, seed=b)
    ms, ctx = results[BATCH][0] * 1e3, results[BATCH][1]
    value = BATCH / results[BATCH][0]
    bytes_step = weight_bytes + BATCH * ctx * kv_per_tok
    achieved = bytes_step / results[BATCH][0] / 1e9

    out = {
        "metric": "decode tokens/s, batch %d, %d-token prompts (MiniCPM-%s-shaped)" % (BATCH, PROMPT, args.shape.upper()),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic (seeded random weights N(0,0.1) and token ids)",
        "config": {
            "model": "MiniCPM-%s-shaped" % args.shape.upper(), "layers": conf.num_hidden_layers, "layers_of_config": MODEL["num_hidden_layers"],
            "hidden": conf.hidden_size, "heads": conf.num_attention_heads, "kv_heads": conf.num_key_value_heads,
            "head_dim": conf.head_dim, "intermediate": conf.intermediate_size, "vocab": conf.vocab_size,
            "global_batch": BATCH, "seq_len": PROMPT, "context_mean": round(ctx, 1), "generated": args.steps,
            "page_size": args.page_size, "tied_embeddings": bool(MODEL.get("tie_word_embeddings", True)), "parallelism": "single-gpu",
            "sampling": "greedy on device", "library_gemm": "default" if args.no_tune else "algorithms timed per shape",
            "decode_launch": "eager" if args.eager else "hip graph", "decode_loop": "direct" if args.direct else "scheduler",
        },
        "prefill": {"value": round(PROMPT / t_pf, 1), "tokens": PROMPT, "ms": round(t_pf * 1e3, 3),
                    "frac": round(pf_flops / t_pf / (PEAK_TFLOPS[dname] * 1e12), 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {("decode_b%d" % b): round(b / results[b][0], 1) for b in batches if b != BATCH},
        # every point's step against the same bound: the bytes it has to read (weights once, the live requests' cache) / its time
        "points_roofline": {("decode_b%d" % b): {
            "ms": round(results[b][0] * 1e3, 4), "context": round(results[b][1], 1),
            "achieved": round((weight_bytes + b * results[b][1] * kv_per_tok) / results[b][0] / 1e9, 1),
            "frac": round((weight_bytes + b * results[b][1] * kv_per_tok) / results[b][0] / 1e9 / HBM_PEAK_GBS, 4)}
            for b in batches},
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
