"""The Fopezen decoder in the engine against the plain implementation of its equations (plain_fopezen.py):
each mechanism's kernel alone, then whole models in the four replay modes, both dtypes, with sizes and
constants chosen so that no two of them coincide, and greedy generation through the entry point."""
import json
import math
import os
import random

import pytest
import torch

import helpers as H
import plain_fopezen as P

pytestmark = pytest.mark.gpu

DTYPES = [("float32", torch.float32, H.FP32_TOL), ("bfloat16", torch.bfloat16, H.BF16_TOL)]


def _layer(kind, heads, kv, dim, vdim, scale, size, keep, v_mix, ff):
    mask = {"size": size, "keep_first": keep} if size else None
    return {"type": kind, "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
                                    "mask": mask, "v_mix": v_mix},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


# F1: sizes of the tiled kernels, values wider than keys, the two mixers in both orders, a layer without a
# feed-forward, a layer that does not mix values between two that do, a layer without a mask.
F1 = {"architecture": "Fopezen", "vocab": 211, "width": 128, "norm": {"eps": 1e-5}, "layers": [
    _layer("attention_2", 4, 2, 32, 64, 0.2, 40, 3, True, 192),
    _layer("attention", 2, 1, 64, 32, 0.11, 24, 0, False, None),
    _layer("attention", 4, 2, 32, 64, 0.15, 56, 9, True, 160),
    _layer("attention_2", 4, 2, 64, 64, 0.09, None, 0, True, 96),
]}
# F2: sizes no tiled kernel takes (the general kernel), one kv head per head, one kept key, a window of one.
F2 = {"architecture": "Fopezen", "vocab": 97, "width": 66, "norm": {"eps": 1e-6}, "layers": [
    _layer("attention", 3, 3, 24, 40, 0.3, 17, 5, True, 100),
    _layer("attention_2", 3, 3, 20, 40, 0.25, 1, 1, True, 70),
    _layer("attention", 1, 1, 48, 8, 0.2, 33, 40, False, 50),
]}
# F3: key and value size 128, eight query heads on one kv head (two walks over the keys when decoding), kept
# keys that span more than one step of 64 keys and several pages, windows across page borders.
F3 = {"architecture": "Fopezen", "vocab": 300, "width": 192, "norm": {"eps": 1e-5}, "layers": [
    _layer("attention", 8, 1, 128, 128, 0.08, 100, 70, True, 256),
    _layer("attention_2", 8, 2, 64, 64, 0.12, 130, 0, False, 256),
    _layer("attention", 8, 1, 32, 128, 0.2, 64, 16, True, None),
]}
# F4: no masks at all (every key is read, nothing is given back: decoding may run a step ahead of the host), no value mixing.
F4 = {"architecture": "Fopezen", "vocab": 150, "width": 64, "norm": {"eps": 1e-5}, "layers": [
    _layer("attention", 2, 2, 32, 32, 0.18, None, 0, False, 96),
    _layer("attention_2", 4, 1, 16, 24, 0.25, None, 0, False, 80),
]}
CONFIGS = {"F1": F1, "F2": F2, "F3": F3, "F4": F4}
LENGTHS = {"F1": [1, 2, 130, 61, 210, 37], "F2": [3, 75, 1, 140, 18, 66], "F3": [5, 260, 129, 64, 331, 2],
           "F4": [2, 90, 17, 1, 133, 40]}


def _write_model(folder, cfg, seed):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    W = P.random_weights(cfg, seed)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return W


_models, _engines, _plain = {}, {}, {}


def _model(tmp_path_factory, name):
    if name not in _models:
        folder = os.path.join(str(tmp_path_factory.getbasetemp()), "fopezen_" + name)
        _models[name] = (folder, _write_model(folder, CONFIGS[name], seed=len(name) + ord(name[-1])))
    return _models[name]


def _engine(tmp_path_factory, name, dtype, max_tokens, page_size=16, attention="auto", max_requests=4):
    from infinicore_infer_amd.engine import Engine
    key = (name, dtype, max_tokens, page_size, attention, max_requests)
    if key not in _engines:
        folder, _ = _model(tmp_path_factory, name)
        _engines[key] = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=page_size,
                                        max_requests=max_requests, attention_impl=attention)
    return _engines[key]


def _requests(name, seed=0):
    return {"r%d" % i: H.random_tokens(CONFIGS[name]["vocab"], n, seed * 100 + i) for i, n in enumerate(LENGTHS[name])}


def _reference(tmp_path_factory, name, requests):
    key = (name, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in _plain:
        _, W = _model(tmp_path_factory, name)
        _plain[key] = {rid: P.forward(CONFIGS[name], W, toks, torch.float64) for rid, toks in requests.items()}
    return _plain[key]


MODES = {
    "whole": H.trace_whole,
    "tail": lambda r: H.trace_last_one_by_one(r, tail=150),     # windows pass over decoded tokens; recorded steps replay
    "chunks": H.trace_chunks,
    "mixed": H.trace_mixed,
}


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_modes(tmp_path_factory, name, dname, dtype, tol, mode):
    """Prefill against token-by-token decoding, portions down to two tokens, unequal requests in one batch with
    pages and state slots used again: every position's logits against the plain implementation."""
    requests = _requests(name)
    steps, max_tokens = MODES[mode](requests)
    engine = _engine(tmp_path_factory, name, dtype, max_tokens)
    ref = _reference(tmp_path_factory, name, requests)
    got = H.run_trace(engine, steps)
    assert len(got) == sum(len(t) for t in requests.values())
    worst = H.compare(got, ref, tol, "%s %s %s" % (name, dname, mode))
    print("worst error %.3g at %s (allowed %.3g)" % (worst[0], worst[1], tol))
    engine.cache.check_invariants()
    assert not engine.cache.requests
    for g in range(len(engine.groups)):
        assert engine.cache.free_pages(g) == engine.num_pages


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name,page_size", [("F1", 64), ("F3", 32), ("F1", 16)])
def test_general_kernel_alone_and_other_page_sizes(tmp_path_factory, name, page_size, dname, dtype, tol):
    requests = _requests(name, seed=2)
    steps, max_tokens = H.trace_mixed(requests, seed=5)
    max_tokens = (max_tokens + 4 * page_size)              # each live request's count is rounded up to whole pages
    ref = _reference(tmp_path_factory, name, requests)
    for attention in ("generic", "auto"):
        engine = _engine(tmp_path_factory, name, dtype, max_tokens, page_size=page_size, attention=attention)
        H.compare(H.run_trace(engine, steps), ref, tol, "%s %s %s page %d" % (name, dname, attention, page_size))
        engine.cache.check_invariants()


def test_recorded_decode_steps_equal_eager_ones(tmp_path_factory):
    """Long decoding: the same request decoded through recorded steps and eagerly gives the same logits."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, _ = _model(tmp_path_factory, "F1")
    toks = H.random_tokens(F1["vocab"], 230, 9)
    rows = {}
    for graphs in (True, False):
        eng = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=512, page_size=16, max_requests=2, use_graphs=graphs)
        eng.step([StepEntry("a", toks[:30], [])])
        out = []
        for t in toks[30:]:
            out.append(eng.step([StepEntry("a", [t], [0])]).float().cpu().clone())
        rows[graphs] = torch.cat(out)
        if graphs:
            assert eng.graph_replays > 100
    assert torch.equal(rows[True], rows[False])


# ---- the mechanisms alone ------------------------------------------------------------------------------------------
def _dev(t, dtype=None):
    return (t if dtype is None else t.to(dtype)).cuda().contiguous()


@pytest.mark.parametrize("width,first", [(64, 0), (130, 1000), (256, 60000), (77, 300)])
def test_embedding_with_position_vector(width, first):
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.parts.embedding import sinusoid_frequencies
    g = torch.Generator().manual_seed(width)
    table = torch.randn(50, width, generator=g).to(torch.bfloat16)
    tokens = torch.randint(0, 50, (37,), generator=g)
    pos = torch.arange(first, first + 37)
    x = torch.empty(37, width, dtype=torch.float32, device="cuda")
    copy = torch.empty(37, width, dtype=torch.bfloat16, device="cuda")
    ops.embed_sinusoid(_dev(tokens, torch.int32), _dev(pos, torch.int32), _dev(table), sinusoid_frequencies(width, 10000.0).cuda(),
                       x, copy=copy)
    assert torch.equal(copy.cpu(), x.cpu().to(torch.bfloat16))
    # far positions too: the angle keeps what the float32 product p * f rounds away
    exact = table.double()[tokens] + P.sinusoid(pos, width, torch.float64)
    assert float((x.cpu().double() - exact).abs().max()) < 2e-6


@pytest.mark.parametrize("d,bias", [(64, False), (200, True), (1026, True)])
def test_norm_into_stream(d, bias):
    from infinicore_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(d)
    y = (torch.randn(19, d, generator=g) * 3).to(torch.bfloat16)
    w = torch.randn(d, generator=g) * 0.1
    b = torch.randn(d, generator=g) if bias else None
    x0 = torch.randn(19, d, generator=g)
    want = x0 + P.norm_one_plus(y.float() + (b if bias else 0.0), w, 1e-5)
    x = _dev(x0)
    copy = torch.empty(19, d, dtype=torch.bfloat16, device="cuda")
    ops.norm_into_stream(_dev(y), _dev(1.0 + w), x, 1e-5, bias=_dev(b) if bias else None, copy=copy)
    assert float((x.cpu() - want).abs().max()) < 1e-5
    assert torch.equal(copy.cpu(), x.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("kind", ["relu2", "gelu_tanh", "silu"])
def test_activations(kind):
    from infinicore_infer_amd.kernels import ops
    z = torch.linspace(-6, 6, 1001)
    want = {"relu2": torch.relu(z) ** 2,
            "gelu_tanh": 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))),
            "silu": z * torch.sigmoid(z)}[kind]
    x = _dev(z)
    ops.activation(x, x, kind)
    assert float((x.cpu() - want).abs().max()) < 1e-5


class _Paged:
    """Keys and values of a few requests in shuffled pages, with block tables (built by hand, not by the engine)."""

    def __init__(self, lens, G, dk, dv, page, dtype, seed, extra_pages=3):
        g = torch.Generator().manual_seed(seed)
        self.k = [torch.randn(n, G, dk, generator=g).to(dtype) for n in lens]
        self.v = [torch.randn(n, G, dv, generator=g).to(dtype) for n in lens]
        need = [(n + page - 1) // page for n in lens]
        ids = list(range(sum(need) + extra_pages))
        random.Random(seed).shuffle(ids)
        # unused pages hold NaN: a kernel that multiplies a masked key's value poisons its result
        self.kc = torch.full((len(ids), G, page, dk), float("nan")).to(dtype)
        self.vc = torch.full((len(ids), G, page, dv), float("nan")).to(dtype)
        self.bt = torch.zeros(len(lens), max(need), dtype=torch.int32)
        self.bt[:] = ids[-1]                                   # entries past a request's pages point at a NaN page
        for r, n in enumerate(lens):
            for j in range(need[r]):
                pg = ids.pop(0)
                self.bt[r, j] = pg
                lo, hi = j * page, min(n, (j + 1) * page)
                self.kc[pg, :, :hi - lo] = self.k[r][lo:hi].transpose(0, 1)
                self.vc[pg, :, :hi - lo] = self.v[r][lo:hi].transpose(0, 1)
                self.kc[pg, :, hi - lo:] = 0                   # the rest of a request's last page: written later, finite
                self.vc[pg, :, hi - lo:] = 0


def _span_reference(q, paged, r, pos0, H_, G, scale, window, keep, sink, gate):
    """Rows of request r at positions pos0.. against the plain attend()."""
    n = q.shape[0]
    T = pos0 + n
    vis = P.visible(T, window, keep)[pos0:]
    k = paged.k[r][:T].double().reshape(T, -1)
    v = paged.v[r][:T].double().reshape(T, -1)
    out = []
    qd = q.double().view(n, H_, -1)
    for h in range(H_):
        gi = h // (H_ // G)
        dk = qd.shape[-1]
        s = (qd[:, h] @ k.view(T, G, dk)[:, gi].T) * scale
        out.append(P.weights_of_scores(s, vis, sink) @ v.view(T, G, -1)[:, gi])
    out = torch.cat(out, -1)
    return out * torch.sigmoid(gate.double()) if gate is not None else out


SPAN_CASES = [
    # H, G, dk, dv, window, keep, sink, gate, page
    (4, 2, 64, 32, 40, 5, True, True, 16),
    (4, 2, 32, 64, 64, 0, False, False, 16),
    (8, 1, 128, 128, 100, 70, True, True, 32),
    (2, 2, 64, 64, 0, 0, False, True, 64),
    (6, 3, 128, 32, 31, 33, True, False, 16),
    (3, 1, 24, 40, 17, 2, True, True, 16),          # sizes only the general kernel takes
]


@pytest.mark.parametrize("dname,dtype,tol", [("float32", torch.float32, 2e-5), ("bfloat16", torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("case", SPAN_CASES)
def test_span_attention_kernels(case, dname, dtype, tol):
    """The general kernel, the split-key kernel (1, 2 and 7 splits) and the matrix-core kernel against the plain
    softmax over the visible keys: prompt portions that start anywhere, single tokens at, just before and just after
    every edge (the window's, the kept keys', a page's), with one key's score made to stand out just inside and just
    outside the window and among the kept keys."""
    from infinicore_infer_amd.kernels import ops
    H_, G, dk, dv, window, keep, sink, use_gate, page = case
    scale = 1.0 / math.sqrt(dk)
    lens = [300, 150, 7]
    pg = _Paged(lens, G, dk, dv, page, dtype, seed=dk + dv + window)
    g = torch.Generator().manual_seed(7)
    kc, vc, bt = pg.kc.cuda(), pg.vc.cuda(), pg.bt.cuda()

    def run(kernel, req_rows):
        """req_rows: [(request, first position, rows)] -> out rows and their reference."""
        qs, refs, gates, token_req, positions, tiles, row = [], [], [], [], [], [], 0
        for r, p0, n in req_rows:
            q = torch.randn(n, H_ * dk, generator=g)
            # a needle: the query of the last row is aligned with one key just inside / outside its window or kept keys
            last = p0 + n - 1
            for target in {max(0, last - window + 1) if window else 0, max(0, last - window) if window else 0,
                           max(0, keep - 1), min(keep, last)}:
                if 0 <= target <= last and random.Random(target + n).random() < 0.6:
                    q[n - 1].view(H_, dk)[:] += 6.0 * pg.k[r][target].float().repeat_interleave(H_ // G, 0)
            q = q.to(dtype)
            gate = torch.randn(n, H_ * dv, generator=g).to(dtype) if use_gate else None
            refs.append(_span_reference(q.float(), pg, r, p0, H_, G, scale, window or None, keep, sink,
                                        gate.float() if use_gate else None))
            qs.append(q)
            gates.append(gate)
            token_req += [r] * n
            positions += list(range(p0, p0 + n))
            for o in range(0, n, 128):
                tiles.append((r, row + o, min(128, n - o), p0 + o))
            row += n
        q = torch.cat(qs).cuda()
        gate = torch.cat(gates).cuda() if use_gate else None
        out = torch.full((row, H_ * dv), float("nan"), dtype=dtype, device="cuda")
        tr, ps_ = torch.tensor(token_req, dtype=torch.int32).cuda(), torch.tensor(positions, dtype=torch.int32).cuda()
        args = (H_, G, dk, dv, page, scale, window, keep, sink)
        if kernel == "general":
            ops.attention_span_generic(q, out, gate, kc, vc, bt, tr, ps_, *args)
        elif kernel == "prefill":
            tl = torch.tensor(tiles, dtype=torch.int32).cuda()
            ops.attention_span_prefill(q, out, gate, kc, vc, bt, tl, len(tiles), *args)
        else:
            ns = int(kernel)
            pa = torch.empty(row * H_ * ns * dv, dtype=torch.float32, device="cuda")
            pm = torch.empty(row * H_ * ns * 2, dtype=torch.float32, device="cuda")
            ops.attention_span_decode(q, out, gate, kc, vc, bt, None, row, tr, ps_, pa, pm, *args, n_split=ns)
        ref = torch.cat(refs)
        err = float((out.float().cpu().double() - ref).abs().max()) / max(1.0, float(ref.abs().max()))
        assert math.isfinite(err) and err <= tol, "%s: error %.3g (allowed %.3g)" % (kernel, err, tol)

    edges = sorted({0, 1, keep - 1, keep, keep + 1, window - 1, window, window + 1, window + keep, page - 1, page, 63, 64, 65,
                    127, 128, 149, 299} - {-1})
    singles = [(0, p, 1) for p in edges if p < 300] + [(1, p, 1) for p in edges if p < 150] + [(2, 6, 1)]
    portions = [(0, 0, 300), (1, 0, 2), (2, 0, 7), (1, 2, 131), (0, 171, 129), (1, 133, 17), (0, 64, 2), (0, 40, 70)]
    run("general", singles + portions)
    if ops.attention_span_decode_supported(dtype, dk, dv):
        for ns in (1, 2, 7):
            run(str(ns), singles)
    else:
        assert dk % 32 or dv % 32
    if ops.attention_span_prefill_supported(dtype, dk, dv):
        run("prefill", portions + singles[:5])
    else:
        assert dtype == torch.float32 or dk % 32 or dv % 32


@pytest.mark.parametrize("mode,mix", [(1, 0), (1, 1), (2, 2), (0, 2), (2, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,G,dk,dv,extra", [(6, 3, 24, 40, 13), (4, 2, 64, 32, 16), (5, 5, 32, 128, 0), (3, 1, 128, 8, 24),
                                              (4, 2, 64, 32, 3), (40, 8, 128, 64, 0)])
def test_bias_norm_value_mix_and_cache_write(mode, mix, dtype, Hq, G, dk, dv, extra):
    """Sizes that take the kernel's 16-byte path (pieces per head a power of two, aligned rows) and sizes that do not."""
    from infinicore_infer_amd.kernels import ops
    page, T = 16, 21
    g = torch.Generator().manual_seed(mode * 3 + mix)
    rows = torch.randn(T, Hq * dk + G * dk + G * dv + extra, generator=g).to(dtype)
    bias = torch.randn(Hq * dk + G * dk + G * dv, generator=g)
    qw = torch.randn(dk if mode == 1 else Hq * dk, generator=g)
    kw = torch.randn(dk if mode == 1 else G * dk, generator=g)
    lam = torch.tensor([0.37])
    keep0 = torch.randn(T, G * dv, generator=g)
    slots = torch.randperm(5 * page, generator=g)[:T].to(torch.int32)
    r = rows.float()
    q = r[:, :Hq * dk] + bias[:Hq * dk]
    k = r[:, Hq * dk:(Hq + G) * dk] + bias[Hq * dk:(Hq + G) * dk]
    v = r[:, (Hq + G) * dk:(Hq + G) * dk + G * dv] + bias[(Hq + G) * dk:]
    if mode == 1:
        q, k = P.qk_norm_per_head(q, qw, Hq, 1e-5), P.qk_norm_per_head(k, kw, G, 1e-5)
    elif mode == 2:
        q, k = P.qk_norm_whole(q, qw, 1e-5), P.qk_norm_whole(k, kw, 1e-5)
    v_cached = P.mix_values(v, keep0, lam) if mix == 2 else v
    kc = torch.zeros(5, G, page, dk, dtype=dtype, device="cuda")
    vc = torch.zeros(5, G, page, dv, dtype=dtype, device="cuda")
    q_out = torch.empty(T, Hq * dk, dtype=dtype, device="cuda")
    v_keep = _dev(keep0)
    ops.qk_norm_store(_dev(rows), _dev(bias), _dev(qw) if mode else None, _dev(kw) if mode else None, mode, 1e-5, mix,
                      _dev(lam) if mix == 2 else None, v_keep if mix else None, q_out, kc, vc, _dev(slots), Hq, G, dk, dv, page)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((q_out.float().cpu() - q).abs().max()) <= tol * float(q.abs().max())
    for t in range(T):
        pgi, off = int(slots[t]) // page, int(slots[t]) % page
        assert float((kc[pgi, :, off].float().cpu().reshape(-1) - k[t]).abs().max()) <= tol * float(k.abs().max())
        assert float((vc[pgi, :, off].float().cpu().reshape(-1) - v_cached[t]).abs().max()) <= tol * float(v.abs().max())
    if mix == 1:
        assert float((v_keep.cpu() - v).abs().max()) < 1e-6 * float(v.abs().max()) + 1e-6


# ---- generation through the entry point ------------------------------------------------------------------------------
def _plain_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(P.forward(cfg, W, toks, torch.float64)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["F1", "F2", "F4"])
def test_greedy_generation_through_the_entry_point_and_scheduler(tmp_path_factory, name):
    """Several prompts of unequal length through CausalLM.generate_batch (the scheduler: chunked prompts, continuous
    batching, recorded decode steps) in float32: the plain implementation's greedy tokens."""
    from infinicore_infer_amd.causal_lm import CausalLM
    folder, W = _model(tmp_path_factory, name)
    cfg = CONFIGS[name]
    prompts = [H.random_tokens(cfg["vocab"], n, 40 + i) for i, n in enumerate([50, 3, 21])]
    model = CausalLM(folder, max_tokens=256, dtype=torch.float32, cache_tokens=1024, page_size=16, max_requests=4)
    outs = model.generate_batch(prompts, 12, max_batch_tokens=24, chunk_size=16)
    for p, o in zip(prompts, outs):
        assert o == _plain_greedy(cfg, W, p, 12)
    model.engine.cache.check_invariants()
    if name == "F4":
        assert model.engine.steps_ahead > 0          # without windows the device fed its own tokens to recorded steps


def test_command_line_runs_the_design(tmp_path_factory):
    """python -m infinicore_infer_amd.causal_lm on a Fopezen folder generates the plain implementation's tokens."""
    import subprocess
    import sys
    folder, W = _model(tmp_path_factory, "F1")
    prompt = H.random_tokens(F1["vocab"], 9, 77)
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.causal_lm", "--amd", folder, "--dtype", "float32",
                        "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--max-tokens", "128"],
                       cwd=H.__file__.rsplit("/tests/", 1)[0], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    want = _plain_greedy(F1, W, prompt, 6)
    assert " ".join(map(str, want)) in " ".join(r.stdout.split()), r.stdout[-2000:]


# ---- configurations drawn from seeds -------------------------------------------------------------------------------------
def _drawn_config(seed):
    """Layer order, sizes (also ones that are no multiple of 8 or 16), windows, kept keys, scales and mixing drawn from a seed."""
    rng = random.Random(seed)
    width = rng.choice([34, 48, 64, 100, 136]) if seed < 10 else [51, 77][seed % 2]      # odd widths too
    kv, vdim = rng.choice([1, 2, 3]), rng.choice([8, 12, 20, 32, 64])        # shared by the mixing layers
    layers = []
    for i in range(rng.choice([2, 3, 4, 5])):
        mixes = rng.random() < 0.6
        g = kv if mixes else rng.choice([1, 2, 4])
        heads = g * rng.choice([1, 2, 3, 5])
        dim = rng.choice([8, 12, 16, 24, 32, 40, 64, 128])
        dv = vdim if mixes else rng.choice([8, 16, 32, 48, 64, 128])
        size = rng.choice([None, 1, 2, 7, 16, 31, 64, 65, 100])
        keep = rng.choice([0, 0, 1, 3, 16, 17, 70]) if size else 0
        ff = rng.choice([None, 24, 50, 128])
        layers.append(_layer(rng.choice(["attention", "attention_2"]), heads, g, dim, dv, round(rng.uniform(0.05, 0.4), 3),
                             size, keep, mixes, ff))
    return {"architecture": "Fopezen", "vocab": rng.choice([53, 128, 301]), "width": width,
            "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])}, "layers": layers}


@pytest.mark.parametrize("seed", list(range(12)))
def test_drawn_configurations(tmp_path_factory, seed):
    from infinicore_infer_amd.engine import Engine
    cfg = _drawn_config(seed)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "fopezen_drawn_%d" % seed)
    W = _write_model(folder, cfg, seed)
    rng = random.Random(seed + 100)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab"], n, seed * 10 + i)
                for i, n in enumerate([rng.choice([1, 2, 5, 40, 66, 129, 180, 250]) for _ in range(5)])}
    ref = {rid: P.forward(cfg, W, toks, torch.float64) for rid, toks in requests.items()}
    steps, max_tokens = H.trace_mixed(requests, seed=seed)
    for dname, dtype, tol in DTYPES:
        engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=16, max_requests=4)
        H.compare(H.run_trace(engine, steps), ref, tol, "drawn %d %s" % (seed, dname), steps)
        engine.cache.check_invariants()
        assert not engine.cache.requests


@pytest.mark.parametrize("kind", ["relu2", "gelu_tanh", "silu"])
@pytest.mark.parametrize("M,N,K", [(1, 384, 256), (8, 14336, 4096), (16, 200, 72), (5, 100000, 64)])
def test_activation_in_the_products_epilogue_equals_the_two_kernels(kind, M, N, K):
    from infinicore_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(M + N)
    a = _dev(torch.randn(M, K, generator=g), torch.bfloat16)
    w = _dev(torch.randn(N, K, generator=g) / math.sqrt(K), torch.bfloat16)
    fused = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    plain = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ops.gemm_nt(a, w, fused, activation=kind)
    ops.gemm_nt(a, w, plain)
    ops.activation(plain, plain, kind)
    assert torch.equal(fused, plain)


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_forked_requests_go_on_independently(tmp_path_factory, dname, dtype, tol):
    """A request's cache (planes of two widths, kept first pages, pages behind the window given back) copied into pages
    of its own; the copy and the original go on with different tokens."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "F1")
    eng = Engine.from_dir(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=4)
    base = H.random_tokens(F1["vocab"], 97, 1)
    tails = {"a": H.random_tokens(F1["vocab"], 30, 2), "b": H.random_tokens(F1["vocab"], 30, 3)}
    eng.step([StepEntry("a", base[:60], [])])
    eng.step([StepEntry("a", base[60:], [])])
    eng.fork("a", "b")
    eng.cache.check_invariants()
    got = {}
    for i in range(30):
        rows = eng.step([StepEntry(r, [tails[r][i]], [0]) for r in ("a", "b")]).float().cpu()
        for j, r in enumerate(("a", "b")):
            got[(r, len(base) + i)] = rows[j].clone()
    ref = {r: P.forward(F1, W, base + tails[r], torch.float64) for r in tails}
    H.compare(got, ref, tol, "fork %s" % dname)
    eng.free("a")
    eng.free("b")
    for g in range(len(eng.groups)):
        assert eng.cache.free_pages(g) == eng.num_pages


def test_command_line_with_random_weights(tmp_path):
    """--random-weights --config: weights drawn for the configuration, several prompts through the scheduler."""
    import subprocess
    import sys
    path = str(tmp_path / "config.json")
    with open(path, "w") as f:
        json.dump(F3, f)
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.fopezen", "--amd", "--random-weights", "--config", path,
                        "--prompt-len", "40", "--num-prompts", "3", "--max-new-tokens", "5", "--max-tokens", "256",
                        "--max-batch-tokens", "64", "--chunk-size", "32", "--weights-norm-std", "0.05"],
                       cwd=H.__file__.rsplit("/tests/", 1)[0], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.count("tokens[") == 3, r.stdout[-2000:]
