"""The Daborax decoder in the engine against the plain implementation of its equations (plain_daborax.py): each
mechanism's kernel alone, then whole models in the four replay modes and both dtypes, with sizes, counts, constants and
layer orders that differ from model to model, and greedy generation through the entry point."""
import json
import math
import os
import random

import pytest
import torch

import helpers as H
import plain_daborax as P

pytestmark = pytest.mark.gpu

DTYPES = [("float32", torch.float32, 2e-4), ("bfloat16", torch.bfloat16, 6e-2)]
BF16_MEAN = 1.5e-2


def _compare(got, ref, dtype, tol, what, steps=None):
    worst = H.compare(got, ref, tol, what, steps)
    if dtype == torch.bfloat16:       # single positions may sit where a norm magnifies rounding; the mean over positions may not
        errs = [float((row.double() - ref[rid][pos]).abs().max()) / float(ref[rid].abs().max()) for (rid, pos), row in got.items()]
        assert sum(errs) / len(errs) <= BF16_MEAN, "%s: mean error %.3g" % (what, sum(errs) / len(errs))
    return worst


def _attention(heads, kv_heads, dim, vdim, scale, window, softcap, ff, limit=2.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def _lightning(heads, dim, vdim, decay, ff, limit=2.0):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay},
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def _mamba(heads, vdim, state, groups, norm_groups, conv, ff, limit=2.0):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups,
                                        "conv": conv}, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def _again(layer, of):
    return dict(json.loads(json.dumps(layer)), weights_of=of)


# D1: key and value sizes of the tiled attention kernels (values wider than keys), a window that is no multiple of a page,
# every kind of layer run twice with the same tensors, in another order the second time.
_d1 = [_attention(4, 2, 32, 64, 0.18, 40, 30.0, 96, 1.0), _lightning(2, 32, 16, [0.9, 0.97], 64, 0.7), _mamba(4, 16, 24, 2, 2, 4, 80, 1.2)]
D1 = {"architecture": "Daborax", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 7.0}, "residual_mult": 0.4,
      "layers": _d1 + [_again(_d1[2], 2), _again(_d1[0], 0), _again(_d1[1], 1)]}
# D2: sizes that only the general kernels take (no multiple of 8), as many kv heads as heads, a window of one token, no
# cap on the scores, one group and one norm group, a convolution of one tap, a layer without a feed-forward, a decay of
# one (nothing forgotten) and of zero (nothing kept), a multiplier and an embedding scale of one.
D2 = {"architecture": "Daborax", "vocab": 97, "width": 70, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "residual_mult": 1.0,
      "layers": [_lightning(3, 10, 12, [1.0, 0.0, 0.5], None), _attention(3, 3, 12, 20, 0.3, 1, None, 50),
                 _mamba(3, 20, 10, 1, 1, 1, 50), _attention(2, 1, 24, 8, 0.25, 17, 5.0, None)]}
# D3: attention over all earlier keys (no mask) beside a window longer than the requests, eight heads on one kv head,
# the layer that lends its tensors comes after the one that borrows them, head size 128.
_d3 = [_attention(8, 1, 128, 32, 0.09, None, 20.0, 64), _lightning(4, 64, 64, [0.5, 0.8, 0.95, 0.999], 128), _attention(2, 2, 64, 64, 0.125, 500, 50.0, 64)]
D3 = {"architecture": "Daborax", "vocab": 300, "width": 128, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0}, "residual_mult": 0.25,
      "layers": [_again(_d3[1], 2), _d3[0], _d3[1], _d3[2], _mamba(2, 64, 16, 2, 4, 3, None)]}
CONFIGS = {"D1": D1, "D2": D2, "D3": D3}
LENGTHS = {"D1": [1, 2, 130, 61, 210, 37], "D2": [3, 75, 1, 140, 18, 66], "D3": [2, 90, 17, 1, 260, 40]}


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
        folder = os.path.join(str(tmp_path_factory.getbasetemp()), "daborax_" + name)
        _models[name] = (folder, _write_model(folder, CONFIGS[name], seed=len(name) + ord(name[-1])))
    return _models[name]


def _engine(tmp_path_factory, name, dtype, max_tokens, page_size=16, max_requests=4):
    from infinicore_infer_amd.engine import Engine
    key = (name, dtype, max_tokens, page_size, max_requests)
    if key not in _engines:
        folder, _ = _model(tmp_path_factory, name)
        _engines[key] = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests)
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
    "tail": lambda r: H.trace_last_one_by_one(r, tail=100),     # long decoding: the windows pass over decoded tokens
    "chunks": H.trace_chunks,
    "mixed": H.trace_mixed,
}


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_modes(tmp_path_factory, name, dname, dtype, tol, mode):
    """Prefill against token-by-token decoding, portions down to two tokens, unequal requests in one batch with pages
    and state slots used again: every position's logits against the plain implementation."""
    requests = _requests(name)
    steps, max_tokens = MODES[mode](requests)
    engine = _engine(tmp_path_factory, name, dtype, max_tokens)
    ref = _reference(tmp_path_factory, name, requests)
    got = H.run_trace(engine, steps)
    assert len(got) == sum(len(t) for t in requests.values())
    worst = _compare(got, ref, dtype, tol, "%s %s %s" % (name, dname, mode))
    print("worst error %.3g at %s (allowed %.3g)" % (worst[0], worst[1], tol))
    engine.cache.check_invariants()
    assert not engine.cache.requests
    for g in range(len(engine.groups)):
        assert engine.cache.free_pages(g) == engine.num_pages


def _misread(monkeypatch, what):
    """One plausible misreading put into the plain implementation."""
    if what == "window one token longer":
        real = P.seen
        monkeypatch.setattr(P, "seen", lambda n, k, window, first=0: real(n, k, None if window is None else window + 1, first))
    elif what == "window one token shorter":
        real = P.seen
        monkeypatch.setattr(P, "seen", lambda n, k, window, first=0: real(n, k, None if window is None else window - 1, first))
    elif what == "no sink":
        real = P.sink_softmax
        monkeypatch.setattr(P, "sink_softmax", lambda s, m, sink, softcap=None: real(s, m, None, softcap))
    elif what == "sink capped and scaled away to zero":
        real = P.sink_softmax
        monkeypatch.setattr(P, "sink_softmax", lambda s, m, sink, softcap=None: real(s, m, 0.0 * sink, softcap))
    elif what == "no cap":
        real = P.sink_softmax
        monkeypatch.setattr(P, "sink_softmax", lambda s, m, sink, softcap=None: real(s, m, sink, None))
    elif what == "query head h on kv head h % kv_heads":
        real = P.window_attention

        def rolled(h, W, p, heads, kv_heads, dim, vdim, scale, softcap, window, eps):
            W = dict(W)
            order = [hd % kv_heads * (heads // kv_heads) + hd // kv_heads for hd in range(heads)]      # (a permutation of the heads)
            W[p + "q"] = W[p + "q"].view(heads, dim, -1)[order].reshape(heads * dim, -1)
            return real(h, W, p, heads, kv_heads, dim, vdim, scale, softcap, window, eps)
        monkeypatch.setattr(P, "window_attention", rolled)
    elif what == "decays of the heads in reverse":
        real = P.lightning_mixer
        monkeypatch.setattr(P, "lightning_mixer", lambda h, W, p, heads, dim, vdim, decay, eps: real(h, W, p, heads, dim, vdim, decay[::-1], eps))
    elif what == "the new key decays too":
        def late(h, W, p, heads, dim, vdim, decay, eps):
            T = h.shape[0]
            q, k = (P.silu(h @ W[p + n].T).reshape(T, heads, dim) for n in "qk")
            v = P.silu(h @ W[p + "v"].T).reshape(T, heads, vdim)
            o = torch.zeros(T, heads, vdim, dtype=h.dtype)
            for hd in range(heads):
                S = torch.zeros(dim, vdim, dtype=h.dtype)
                for t in range(T):
                    S = decay[hd] * (S + torch.outer(k[t, hd], v[t, hd]))
                    o[t, hd] = S.T @ q[t, hd]
            o = P.unit_rms(o.reshape(T, heads * vdim), eps) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
            return o @ W[p + "o"].T
        monkeypatch.setattr(P, "lightning_mixer", late)
    elif what == "layer scale left out":
        real = P.forward

        def unscaled(cfg, W, tokens, dtype=torch.float64, layers_out=None):
            return real(cfg, {k: (torch.ones_like(v) if k.endswith((".ls1", ".ls2")) else v) for k, v in W.items()}, tokens, dtype, layers_out)
        monkeypatch.setattr(P, "forward", unscaled)
    elif what == "up branch not clamped":
        def loose(h, W, p, limit):
            g = torch.clamp(h @ W[p + "gate"].T, max=limit)
            return (g * torch.sigmoid(1.702 * g) * (h @ W[p + "up"].T + 1.0)) @ W[p + "down"].T
        monkeypatch.setattr(P, "clamped_glu", loose)
    elif what == "two borrowing layers in the other order":
        real = P.forward
        monkeypatch.setattr(P, "forward", lambda cfg, W, tokens, dtype=torch.float64, layers_out=None: real(
            dict(cfg, layers=cfg["layers"][:3] + [cfg["layers"][4], cfg["layers"][3]] + cfg["layers"][5:]), W, tokens, dtype, layers_out))
    else:
        raise ValueError(what)


@pytest.mark.parametrize("what", ["window one token longer", "window one token shorter", "no sink", "sink capped and scaled away to zero",
                                  "no cap", "query head h on kv head h % kv_heads", "decays of the heads in reverse",
                                  "the new key decays too", "layer scale left out", "up branch not clamped",
                                  "two borrowing layers in the other order"])
def test_a_misreading_of_the_design_shows(tmp_path_factory, monkeypatch, what):
    """The comparison the other tests rest on is sharp enough: with one misreading in the plain implementation the float32
    engine no longer agrees with it (the same request agrees without)."""
    folder, W = _model(tmp_path_factory, "D1")
    toks = H.random_tokens(D1["vocab"], 120, 21)
    engine = _engine(tmp_path_factory, "D1", torch.float32, 128)
    steps, _ = H.trace_whole({"a": toks})
    got = H.run_trace(engine, steps)
    H.compare(got, {"a": P.forward(D1, W, toks, torch.float64)}, 2e-4, "as designed")
    _misread(monkeypatch, what)
    with pytest.raises(AssertionError):
        H.compare(got, {"a": P.forward(D1, W, toks, torch.float64)}, 2e-4, what)


def test_the_residual_stream_after_every_layer(tmp_path_factory):
    """Layer by layer in float32, a layer that runs twice counted each time: the stream after every entry of the run order."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "D1")
    toks = H.random_tokens(D1["vocab"], 45, 3)
    want = []
    P.forward(D1, W, toks, torch.float64, layers_out=want)
    eng = Engine.from_dir(folder, dtype=torch.float32, max_tokens=64, max_requests=1)
    got, build = [], eng._build_context

    def probed(entries, starts):
        ctx = build(entries, starts)
        ctx.layer_probe = lambda i, x, pending: got.append(x.clone())
        return ctx
    eng._build_context = probed
    eng.step([StepEntry("a", toks, [])])
    assert len(got) == len(D1["layers"]) + 1
    for i, w in enumerate(want):
        assert torch.allclose(got[i].cpu().double(), w, atol=2e-5 * float(w.abs().max())), "after layer run %d" % i


@pytest.mark.parametrize("name,page_size", [("D1", 64), ("D3", 32)])
def test_other_page_sizes(tmp_path_factory, name, page_size):
    requests = _requests(name, seed=2)
    steps, max_tokens = H.trace_mixed(requests, seed=5)
    ref = _reference(tmp_path_factory, name, requests)
    engine = _engine(tmp_path_factory, name, torch.float32, max_tokens + 4 * page_size, page_size=page_size)
    H.compare(H.run_trace(engine, steps), ref, 2e-4, "%s page %d" % (name, page_size))
    engine.cache.check_invariants()


def test_recorded_decode_steps_equal_eager_ones(tmp_path_factory):
    """Long decoding past the window: the same request decoded through recorded steps and eagerly gives the same logits;
    the states move on exactly once per step, also in the step that is recorded."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "D1")
    toks = H.random_tokens(D1["vocab"], 200, 9)
    rows = {}
    for graphs in (True, False):
        eng = Engine.from_dir(folder, dtype=torch.float32, max_tokens=512, page_size=16, max_requests=2, use_graphs=graphs)
        eng.step([StepEntry("a", toks[:30], [])])
        out = []
        for t in toks[30:]:
            out.append(eng.step([StepEntry("a", [t], [0])]).float().cpu().clone())
        rows[graphs] = torch.cat(out)
        if graphs:
            assert eng.graph_replays > 100
    assert torch.equal(rows[True], rows[False])
    ref = P.forward(D1, W, toks, torch.float64)[30:]
    assert float((rows[True].double() - ref).abs().max()) <= 2e-4 * float(ref.abs().max())


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_forked_requests_go_on_independently(tmp_path_factory, dname, dtype, tol):
    """Pages, recurrent states and convolution inputs are copied; both go on with different tokens."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "D1")
    eng = Engine.from_dir(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=4)
    base = H.random_tokens(D1["vocab"], 97, 1)
    tails = {"a": H.random_tokens(D1["vocab"], 20, 2), "b": H.random_tokens(D1["vocab"], 20, 3)}
    eng.step([StepEntry("a", base[:60], [])])
    eng.step([StepEntry("a", base[60:], [])])
    eng.fork("a", "b")
    got = {}
    for i in range(20):
        rows = eng.step([StepEntry(r, [tails[r][i]], [0]) for r in ("a", "b")]).float().cpu()
        for j, r in enumerate(("a", "b")):
            got[(r, len(base) + i)] = rows[j].clone()
    ref = {r: P.forward(D1, W, base + tails[r], torch.float64) for r in tails}
    _compare(got, ref, dtype, tol, "fork %s" % dname)
    eng.free("a")
    eng.free("b")
    eng.cache.check_invariants()


# ---- the mechanisms alone ------------------------------------------------------------------------------------------
def _dev(t, dtype=None):
    return t.to(device="cuda", dtype=dtype if dtype is not None else t.dtype).contiguous()


def _i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device="cuda")


def test_embedding_scale_and_position_vector():
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.parts.embedding import sinusoid_frequencies
    V, d, scale = 50, 38, 5.5
    g = torch.Generator().manual_seed(0)
    table = torch.randn(V, d, generator=g)
    toks, pos = [3, 49, 0, 7, 7], [0, 1, 511, 4097, 60000]
    out = torch.empty(len(toks), d, dtype=torch.float32, device="cuda")
    ops.embed_sinusoid(_i32(toks), _i32(pos), _dev(table), sinusoid_frequencies(d, 10000.0).cuda(), out, scale=scale)
    for i, (t, p) in enumerate(zip(toks, pos)):
        want = table[t].double() * scale + P.position_vectors(1, d, torch.float64, first=p)[0]
        # (the float32 product p * f alone would be off by 4e-3 at position 60,000: the kernel keeps what it rounds away)
        assert torch.allclose(out[i].cpu().double(), want, atol=4e-6)


def test_norm_with_layer_scale_and_multiplier_into_the_stream():
    """x += m * rms(y + bias) * w * ls through the norm part: the three factors are one vector for the kernel."""
    from infinicore_infer_amd.parts import Runtime
    from infinicore_infer_amd.parts.norm import RMSNorm
    T, d, eps, mult = 5, 70, 1e-6, 0.3
    g = torch.Generator().manual_seed(1)
    x, y, b = torch.randn(T, d, generator=g), 3 * torch.randn(T, d, generator=g), torch.randn(d, generator=g)
    w, ls = 1 + 0.2 * torch.randn(d, generator=g), 0.5 + torch.rand(d, generator=g)
    part = RMSNorm("", Runtime(torch.float32, "cuda"), d, eps, tensor="n", scale_tensor="s", out_mult=mult)
    assert set(part.weight_specs()) == {"n", "s"}
    part.load_weights({"n": _dev(w), "s": _dev(ls)})
    xs = _dev(x)
    part.forward_into_stream(_dev(y), xs, bias=_dev(b))
    want = x.double() + mult * P.unit_rms(y.double() + b.double(), eps) * w.double() * ls.double()
    assert torch.allclose(xs.cpu().double(), want, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_clamped_gated_unit(dtype):
    """Gates above the limit, up values beyond it on both sides, and values well inside."""
    from infinicore_infer_amd.kernels import ops
    T, di, limit, alpha = 6, 40, 1.5, 1.702
    g = torch.Generator().manual_seed(2)
    gu = (3 * torch.randn(T, 2 * di, generator=g)).to(dtype)
    gu[0, :4] = torch.tensor([1.5, 1.51, -9.0, 40.0]).to(dtype)
    gu[0, di:di + 4] = torch.tensor([-1.5, -1.6, 1.5, 77.0]).to(dtype)
    gt, up = torch.clamp(gu[:, :di].double(), max=limit), torch.clamp(gu[:, di:].double(), -limit, limit)
    want = gt * torch.sigmoid(alpha * gt) * (up + 1)
    out = torch.empty(T, di, dtype=dtype, device="cuda")
    ops.glu_clamped(_dev(gu), out, limit, alpha)
    assert torch.allclose(out.cpu().double(), want, atol=1e-5 if dtype == torch.float32 else 2e-2)
    odd = torch.empty(T, di - 1, dtype=dtype, device="cuda")           # a width the 16-byte path does not take
    gu2 = torch.cat([gu[:, :di - 1], gu[:, di:2 * di - 1]], 1)
    ops.glu_clamped(_dev(gu2), odd, limit, alpha)
    assert torch.allclose(odd.cpu().double(), want[:, :di - 1], atol=1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("M,K,di", [(1, 96, 40), (8, 256, 128), (16, 200, 72), (3, 4096, 1024), (24, 512, 256), (32, 1024, 512)])
def test_bounded_gated_unit_as_the_epilogue_of_the_gate_up_product(M, K, di):
    """Few rows: the unit rides in the product's epilogue (both projections rounded to bfloat16 first, as when stored)."""
    from infinicore_infer_amd.kernels import ops
    limit, slope = 1.2, 1.702
    g = torch.Generator().manual_seed(M + di)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (2.5 * torch.randn(2 * di, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    if not ops.rule_gate_up_fused(torch.bfloat16, M, _dev(a), _dev(w), False):
        assert M > 16
        pytest.skip("these operands take the library product and the unit's own kernel")
    gu = (a.double() @ w.double().T).to(torch.bfloat16).double()
    gt, up = torch.clamp(gu[:, :di], max=limit), torch.clamp(gu[:, di:], -limit, limit)
    want = gt * torch.sigmoid(slope * gt) * (up + 1)
    assert float((gu[:, :di] > limit).double().mean()) > 0.02 and float((gu[:, di:].abs() > limit).double().mean()) > 0.05
    out = torch.empty(M, di, dtype=torch.bfloat16, device="cuda")
    ops.gemm_nt(_dev(a), _dev(w), out, swiglu_output=True, glu_clamped=(limit, slope))
    assert torch.allclose(out.cpu().double(), want, atol=3e-2, rtol=2e-2)


def test_norm_then_weight_then_sigmoid_gate():
    from infinicore_infer_amd.kernels import ops
    T, n, eps = 5, 60, 1e-5
    g = torch.Generator().manual_seed(2)
    y, z, w = 4 * torch.randn(T, n, generator=g), torch.randn(T, n + 4, generator=g), 1 + 0.2 * torch.randn(n, generator=g)
    for groups in (1, 3):
        want = P.unit_rms(y.double().view(T, groups, n // groups), eps).reshape(T, n) * w.double() * torch.sigmoid(z[:, 4:].double())
        out = torch.empty(T, n, dtype=torch.float32, device="cuda")
        ops.gated_group_norm(y.cuda(), z.cuda()[:, 4:], w.cuda(), groups, eps, out, gate_after=True)
        assert torch.allclose(out.cpu().double(), want, atol=1e-5)


@pytest.mark.parametrize("chunk_len", [0, 1, 5])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dk,dv", [(3, 10, 12), (2, 64, 64), (4, 32, 16), (1, 128, 128), (2, 24, 200)])
def test_linear_attention_with_a_decay_per_head(heads, dk, dv, dtype, chunk_len):
    """(chunk_len > 0: every portion cut into chunks that run side by side.)  Queries, keys and values read from the
    projection's own rows [v | k | q | gate] with their silu; the matrix state per head carried in its slot between
    portions of 1, 2 and more tokens, beside another sequence, in a slot that is used again; decays of one and zero."""
    from infinicore_infer_amd.kernels import ops
    nq, nv = heads * dk, heads * dv
    g = torch.Generator().manual_seed(heads + dk)
    decay = ([1.0, 0.0, 0.9, 0.999] * 2)[:heads]
    seqs = {r: torch.randn(n, 2 * nq + 2 * nv, generator=g).to(dtype) for r, n in ((0, 40), (1, 9), (2, 6))}
    want = {}
    for r, rows in seqs.items():
        a = P.silu(rows.double())
        v, k, q = a[:, :nv].view(-1, heads, dv), a[:, nv:nv + nq].view(-1, heads, dk), a[:, nv + nq:nv + 2 * nq].view(-1, heads, dk)
        S, out = torch.zeros(heads, dk, dv, dtype=torch.float64), []
        for t in range(len(rows)):
            for h in range(heads):
                S[h] = decay[h] * S[h] + torch.outer(k[t, h], v[t, h])
            out.append(torch.stack([S[h].T @ q[t, h] for h in range(heads)]).reshape(-1))
        want[r] = torch.stack(out)
    state = torch.zeros(3, 7 + heads * dk * dv, dtype=torch.float32, device="cuda")
    dec = torch.tensor(decay, dtype=torch.float32, device="cuda")
    at = {0: 0, 1: 0, 2: 0}
    steps = [[(0, 1, 2)], [(1, 2, 0), (0, 7, 2)], [(0, 2, 2), (1, 1, 0)], [(0, 30, 2), (1, 6, 0)], "free0", [(2, 2, 0)], [(2, 4, 0)]]
    for step in steps:
        if step == "free0":
            state[0].zero_()
            continue
        T = sum(n for _, n, _ in step)
        rows = torch.cat([seqs[r][at[r]:at[r] + n] for r, n, _ in step]).cuda()
        starts = [0]
        for _, n, _ in step:
            starts.append(starts[-1] + n)
        o = torch.empty(T, nv, dtype=torch.float32, device="cuda")
        chunks = None
        if chunk_len:
            most = max((n + chunk_len - 1) // chunk_len for _, n, _ in step)
            chunks = (chunk_len, most, torch.full((len(step) * most * heads * dk * dv,), float("nan"), device="cuda"),
                      torch.full((len(step) * most * heads,), float("nan"), device="cuda"))
        ops.ssm_scan(rows, None, None, dec, None, heads, dv, dk, heads, o, state, 7, _i32(starts), _i32([s for _, _, s in step]),
                     len(step), chunks=chunks, in_act="silu")
        i = 0
        for r, n, _ in step:
            w = want[r][at[r]:at[r] + n]
            assert torch.allclose(o[i:i + n].cpu().double(), w, atol=1e-4 * max(1.0, float(w.abs().max())), rtol=1e-5), (r, at[r], n)
            i += n
            at[r] += n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,G,dk,dv,extra", [(6, 3, 24, 40, 13), (4, 2, 64, 32, 16), (3, 1, 128, 8, 24)])
def test_query_and_key_norm_without_weights(dtype, Hq, G, dk, dv, extra):
    """Bias, then every head of q and k to unit root mean square with no weight; k and v land in their pages."""
    from infinicore_infer_amd.kernels import ops
    T, page, eps = 9, 16, 1e-6
    g = torch.Generator().manual_seed(dk)
    n = (Hq + G) * dk + G * dv
    rows = (2 * torch.randn(T, n + extra, generator=g)).to(dtype)
    bias = torch.randn(n, generator=g)
    kc = torch.zeros(4, G, page, dk, dtype=dtype, device="cuda")
    vc = torch.zeros(4, G, page, dv, dtype=dtype, device="cuda")
    slots = [33, 34, 35, 2, 47, 48, 16, 0, 63]
    q_out = torch.empty(T, Hq * dk, dtype=dtype, device="cuda")
    ops.qk_norm_store(_dev(rows), _dev(bias), None, None, 1, eps, 0, None, None, q_out, kc, vc, _i32(slots), Hq, G, dk, dv, page)
    full = rows[:, :n].double() + bias.double()
    q = P.unit_rms(full[:, :Hq * dk].view(T, Hq, dk), eps).reshape(T, -1)
    k = P.unit_rms(full[:, Hq * dk:(Hq + G) * dk].view(T, G, dk), eps)
    v = full[:, (Hq + G) * dk:].view(T, G, dv)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(q_out.cpu().double(), q, atol=tol)
    for t, s in enumerate(slots):
        assert torch.allclose(kc[s // page, :, s % page].cpu().double(), k[t], atol=tol)
        assert torch.allclose(vc[s // page, :, s % page].cpu().double(), v[t], atol=tol * 4)


class _Paged:
    """Keys and values of several requests laid out in shuffled pages; unused pages hold NaN."""

    def __init__(self, lens, G, dk, dv, page, dtype, seed, extra_pages=3):
        g = torch.Generator().manual_seed(seed)
        self.k = [torch.randn(n, G, dk, generator=g).to(dtype) for n in lens]
        self.v = [torch.randn(n, G, dv, generator=g).to(dtype) for n in lens]
        need = [(n + page - 1) // page for n in lens]
        ids = list(range(sum(need) + extra_pages))
        random.Random(seed).shuffle(ids)
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


ATTENTION_CASES = [
    # heads, kv heads, dk, dv, window, cap, page
    (4, 2, 64, 32, 40, 30.0, 16),
    (4, 2, 32, 64, 64, 0.0, 16),
    (8, 1, 128, 128, 100, 8.0, 32),
    (2, 2, 64, 64, 0, 50.0, 64),
    (6, 3, 128, 32, 31, 2.0, 16),
    (3, 1, 24, 40, 17, 10.0, 16),          # sizes only the general kernel takes
]


@pytest.mark.parametrize("dname,dtype,tol", [("float32", torch.float32, 2e-5), ("bfloat16", torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("case", ATTENTION_CASES)
def test_capped_scores_and_learned_sinks_in_the_attention_kernels(case, dname, dtype, tol):
    """The general kernel, the split-key kernel (1, 2 and 7 splits) and the matrix-core kernel against the plain softmax
    with the cap and one learned sink per head: prompt portions that start anywhere, single tokens at, just before and
    just after every edge (the window's, a page's, a 64-key step's), with one key's score made to stand out just inside
    and just outside the window (large enough that the cap flattens it), sinks well above and well below the scores."""
    from infinicore_infer_amd.kernels import ops
    H_, G, dk, dv, window, cap, page = case
    scale = 1.7 / math.sqrt(dk)
    lens = [300, 150, 7]
    pg = _Paged(lens, G, dk, dv, page, dtype, seed=dk + dv + window)
    g = torch.Generator().manual_seed(7)
    kc, vc, bt = pg.kc.cuda(), pg.vc.cuda(), pg.bt.cuda()
    sinks = torch.tensor(([6.0, -3.0, 0.5, 12.0] * 2)[:H_])

    def run(kernel, req_rows):
        qs, refs, token_req, positions, tiles, row = [], [], [], [], [], 0
        for r, p0, n in req_rows:
            q = torch.randn(n, H_ * dk, generator=g)
            last = p0 + n - 1
            for target in {max(0, last - window + 1) if window else 0, max(0, last - window) if window else 0}:
                if 0 <= target <= last and random.Random(target + n).random() < 0.7:
                    q[n - 1].view(H_, dk)[:] += 6.0 * pg.k[r][target].float().repeat_interleave(H_ // G, 0)
            q = q.to(dtype)
            T = p0 + n
            mask = P.seen(n, T, window or None, first=p0)
            out = []
            for h in range(H_):
                gi = h // (H_ // G)
                s = (q.double().view(n, H_, dk)[:, h] @ pg.k[r][:T, gi].double().T) * scale
                out.append(P.sink_softmax(s, mask, sinks[h].double(), cap or None) @ pg.v[r][:T, gi].double())
            refs.append(torch.cat(out, -1))
            qs.append(q)
            token_req += [r] * n
            positions += list(range(p0, p0 + n))
            for o in range(0, n, 128):
                tiles.append((r, row + o, min(128, n - o), p0 + o))
            row += n
        q = torch.cat(qs).cuda()
        out = torch.full((row, H_ * dv), float("nan"), dtype=dtype, device="cuda")
        tr, ps_ = _i32(token_req), _i32(positions)
        args = (H_, G, dk, dv, page, scale, window, 0, sinks.cuda(), cap)
        if kernel == "general":
            ops.attention_span_generic(q, out, None, kc, vc, bt, tr, ps_, *args)
        elif kernel == "prefill":
            ops.attention_span_prefill(q, out, None, kc, vc, bt, _i32(sum(map(list, tiles), [])), len(tiles), *args)
        else:
            ns = int(kernel)
            pa = torch.empty(row * H_ * ns * dv, dtype=torch.float32, device="cuda")
            pm = torch.empty(row * H_ * ns * 2, dtype=torch.float32, device="cuda")
            ops.attention_span_decode(q, out, None, kc, vc, bt, None, row, tr, ps_, pa, pm, *args, n_split=ns)
        ref = torch.cat(refs)
        err = float((out.float().cpu().double() - ref).abs().max()) / max(1.0, float(ref.abs().max()))
        assert math.isfinite(err) and err <= tol, "%s: error %.3g (allowed %.3g)" % (kernel, err, tol)

    edges = sorted({0, 1, window - 2, window - 1, window, window + 1, page - 1, page, 63, 64, 65, 127, 128, 149, 299} - {-1, -2})
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


# ---- generation through the entry point --------------------------------------------------------------------------------
def _plain_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(P.forward(cfg, W, toks, torch.float64)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["D1", "D2", "D3"])
def test_greedy_generation_through_the_entry_point_and_scheduler(tmp_path_factory, name):
    """Several prompts of unequal length through CausalLM.generate_batch (the scheduler: chunked prompts, continuous
    batching, recorded decode steps) in float32: the plain implementation's tokens."""
    from infinicore_infer_amd.causal_lm import CausalLM
    folder, W = _model(tmp_path_factory, name)
    cfg = CONFIGS[name]
    prompts = [H.random_tokens(cfg["vocab"], n, 40 + i) for i, n in enumerate([50, 3, 21])]
    model = CausalLM(folder, max_tokens=256, dtype=torch.float32, cache_tokens=1024, page_size=16, max_requests=4)
    outs = model.generate_batch(prompts, 10, max_batch_tokens=24, chunk_size=16)
    for p, o in zip(prompts, outs):
        assert o == _plain_greedy(cfg, W, p, 10)
    model.engine.cache.check_invariants()


def test_command_line_runs_the_design(tmp_path_factory):
    import subprocess
    import sys
    folder, W = _model(tmp_path_factory, "D2")
    prompt = H.random_tokens(D2["vocab"], 9, 77)
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.daborax", "--amd", folder, "--dtype", "float32",
                        "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--max-tokens", "128"],
                       cwd=H.__file__.rsplit("/tests/", 1)[0], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    want = _plain_greedy(D2, W, prompt, 6)
    assert " ".join(map(str, want)) in " ".join(r.stdout.split()), r.stdout[-2000:]


def test_command_line_with_random_weights(tmp_path):
    import subprocess
    import sys
    path = str(tmp_path / "config.json")
    with open(path, "w") as f:
        json.dump(D3, f)
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.causal_lm", "--amd", "--random-weights", "--config", path,
                        "--prompt-len", "40", "--num-prompts", "3", "--max-new-tokens", "5", "--max-tokens", "256",
                        "--max-batch-tokens", "64", "--chunk-size", "32", "--weights-norm-std", "0.05"],
                       cwd=H.__file__.rsplit("/tests/", 1)[0], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.count("tokens[") == 3, r.stdout[-2000:]


def test_trace_runner_as_a_program(tmp_path_factory, tmp_path):
    """bin/trace_run on a model folder: steps on standard input, logits files and 'done' lines out; a request left out of
    a step goes on later; pages and the state slots are used again."""
    import subprocess
    folder, W = _model(tmp_path_factory, "D2")
    requests = _requests("D2", seed=4)
    steps, max_tokens = H.trace_mixed(requests, seed=3)
    root = H.__file__.rsplit("/tests/", 1)[0]
    out = str(tmp_path / "out")
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out,
                        "--max-tokens", str(max_tokens)], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.split("\n") if l.startswith("done")] == ["done %d" % s["step"] for s in steps]
    ref = {rid: P.forward(D2, W, toks, torch.float64) for rid, toks in requests.items()}
    at, got = {}, {}
    for s in steps:
        rows = torch.frombuffer(bytearray(open(os.path.join(out, "%d.f32" % s["step"]), "rb").read()), dtype=torch.float32).view(-1, D2["vocab"])
        i = 0
        for e in s["entries"]:
            for w in e["want"]:
                got[(e["id"], at.get(e["id"], 0) + w)] = rows[i].clone()
                i += 1
            at[e["id"]] = at.get(e["id"], 0) + len(e["tokens"])
        assert i == rows.shape[0]
    H.compare(got, ref, 2e-4, "trace runner", steps)


# ---- configurations drawn from seeds -------------------------------------------------------------------------------------
def _drawn_config(seed):
    rng = random.Random(seed)
    width = rng.choice([34, 48, 64, 100])
    layers = []
    for _ in range(rng.choice([2, 3, 4])):
        kind = rng.choice(["attention", "lightning", "mamba2"])
        ff = rng.choice([None, 24, 50, 128])
        limit = rng.choice([0.5, 1.5, 7.0])
        if kind == "lightning":
            heads = rng.choice([1, 2, 3, 5])
            layers.append(_lightning(heads, rng.choice([4, 12, 32, 64]), rng.choice([8, 20, 32, 64]),
                                     [round(rng.choice([0.0, 0.3, 0.9, 0.99, 1.0, rng.uniform(0.5, 1.0)]), 4) for _ in range(heads)], ff, limit))
        elif kind == "mamba2":
            groups = rng.choice([1, 2, 3])
            heads = groups * rng.choice([1, 2])
            vdim = rng.choice([8, 12, 32])
            ng = rng.choice([g for g in (1, 2, 3, 4, 6) if (heads * vdim) % g == 0 and heads * vdim // g >= 8])
            layers.append(_mamba(heads, vdim, rng.choice([4, 9, 16, 40]), groups, ng, rng.choice([1, 2, 3, 4]), ff, limit))
        else:
            kv = rng.choice([1, 2, 3])
            layers.append(_attention(kv * rng.choice([1, 2, 4]), kv, rng.choice([8, 12, 32, 64]), rng.choice([4, 20, 32, 64]),
                                     round(rng.uniform(0.05, 0.4), 3), rng.choice([None, 1, 2, 15, 16, 33, 100]),
                                     rng.choice([None, 1.0, 10.0, 50.0]), ff, limit))
    for i in range(rng.choice([0, 1, 2, 3])):                  # layers that run with another's tensors, put anywhere
        src = rng.randrange(len(layers))
        while layers[src].get("weights_of") is not None:
            src = layers[src]["weights_of"]
        at = rng.randrange(len(layers) + 1)
        layers.insert(at, None)
        for l in layers:                                       # the insertion moves the layers behind it
            if l is not None and l.get("weights_of") is not None and l["weights_of"] >= at:
                l["weights_of"] += 1
        layers[at] = _again(layers[src + (src >= at)], src + (src >= at))
    return {"architecture": "Daborax", "vocab": rng.choice([53, 128, 301]), "width": width, "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])},
            "embedding": {"scale": rng.choice([1.0, 4.0, 11.0])}, "residual_mult": rng.choice([1.0, 0.5, 0.2]), "layers": layers}


@pytest.mark.parametrize("seed", list(range(10)))
def test_drawn_configurations(tmp_path_factory, seed):
    from infinicore_infer_amd.engine import Engine
    cfg = _drawn_config(seed)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "daborax_drawn_%d" % seed)
    W = _write_model(folder, cfg, seed)
    rng = random.Random(seed + 100)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab"], n, seed * 10 + i)
                for i, n in enumerate([rng.choice([1, 2, 5, 40, 66, 129, 150]) for _ in range(5)])}
    ref = {rid: P.forward(cfg, W, toks, torch.float64) for rid, toks in requests.items()}
    steps, max_tokens = H.trace_mixed(requests, seed=seed)
    for dname, dtype, tol in DTYPES:
        engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=16, max_requests=4)
        _compare(H.run_trace(engine, steps), ref, dtype, tol if dtype == torch.float32 else 0.3, "drawn %d %s" % (seed, dname), steps)
        engine.cache.check_invariants()
        assert not engine.cache.requests
