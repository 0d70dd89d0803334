"""The Fizelix decoder in the engine against the plain implementation of its equations (plain_fizelix.py): each
mechanism's kernel alone, then whole models in the four replay modes and both dtypes, with sizes, counts, constants and
layer orders that differ from model to model, and greedy generation through the entry point."""
import json
import math
import os
import random

import pytest
import torch

import helpers as H
import plain_fizelix as P

pytestmark = pytest.mark.gpu

DTYPES = [("float32", torch.float32, 2e-4), ("bfloat16", torch.bfloat16, 8e-2)]
BF16_MEAN = 4e-2
BF16_MEDIAN = 2e-2


def _compare(got, ref, dtype, tol, what, steps=None, loose=False):
    """float32: every position within ``tol`` of the largest logit (``loose``, for configurations drawn at random: all but
    one in a hundred, and none beyond five times that; a position where values nearly cancel before a norm magnifies
    rounding).  bfloat16: the median and the mean over positions, and all but a few positions within ``tol``: where two
    experts' scores lie closer than 16-bit rounding the choice may fall the other way and move that token's row, which with
    four experts of sixteen happens to several positions in a hundred (every position is held to the float32 tolerance in
    the float32 mode, which runs the same steps, and the 16-bit kernels are held to theirs one by one)."""
    if dtype == torch.float32 and not loose:
        return H.compare(got, ref, tol, what, steps)
    H.compare(got, ref, 5 * tol if dtype == torch.float32 else 1e9, what, steps)        # every wanted place is there and finite
    errs = sorted(float((row.double() - ref[rid][pos]).abs().max()) / float(ref[rid].abs().max()) for (rid, pos), row in got.items())
    over = sum(e > tol for e in errs)
    if dtype == torch.float32:
        assert over <= max(1, 0.01 * len(errs)), "%s: %d of %d positions beyond %.3g" % (what, over, len(errs), tol)
        return errs[-1], None
    assert over <= max(1, 0.15 * len(errs)), "%s: %d of %d positions beyond %.3g" % (what, over, len(errs), tol)
    assert errs[len(errs) // 2] <= BF16_MEDIAN, "%s: median error %.3g" % (what, errs[len(errs) // 2])
    mean_most = BF16_MEAN * (1.5 if loose else 1.0)         # (drawn widths go down to 34, where 16-bit rounding weighs more)
    assert sum(errs) / len(errs) <= mean_most, "%s: mean error %.3g" % (what, sum(errs) / len(errs))
    return errs[-1], None


def _dev(t):
    return t.cuda()


def _i32(v):
    return torch.tensor(list(v), dtype=torch.int32, device="cuda")


def _dense(ff):
    return {"kind": "dense", "ff": ff} if ff else None


def _moe(experts, top, ff, shared):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def _attention(heads, kv_heads, dim, vdim, scale, window, pool, rot_dims, rot_base, mlp):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
        if pool:
            m["mask"]["pool"] = pool
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": rot_base}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _mamba(heads, vdim, state, groups, norm_groups, conv, mlp):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups,
                                        "conv": conv}, "mlp": mlp}


# F1: key and value sizes that differ, a window and a block that are no multiple of a page, two experts of four with a shared
# one, the first two layers three times in a row (the loop starts at layer 0), a token input of eight columns per layer.
F1 = {"architecture": "Fizelix", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0}, "logit_scale": 0.5,
      "token_side": {"dim": 8}, "loop": {"start": 0, "stop": 2, "times": 3},
      "layers": [_attention(4, 2, 32, 64, 0.18, 24, 8, 16, 10000.0, _dense(80)),
                 _mamba(4, 16, 24, 2, 2, 4, _moe(4, 2, 48, 64)),
                 _attention(6, 3, 16, 16, 0.3, 33, 5, 16, 500.0, _moe(3, 1, 40, None))]}
# F2: sizes that are no multiple of 8, as many kv heads as heads, a window of one token with blocks of one token (every
# earlier token is then seen as its own block), every entry of a head rotated, a block longer than the window, a layer
# without rotation, a convolution of one tap, a layer without a feed-forward, three experts of five, no loop, no token
# input, scales of one.
F2 = {"architecture": "Fizelix", "vocab": 97, "width": 70, "norm": {"eps": 1e-6},
      "layers": [_attention(3, 3, 10, 12, 0.3, 1, 1, 10, 77.0, _dense(50)),
                 _mamba(3, 20, 10, 1, 1, 1, None),
                 _attention(2, 1, 24, 8, 0.25, 17, 20, 0, None, _moe(5, 3, 30, None))]}
# F3: attention over all earlier tokens (no mask) beside a window longer than the requests, eight heads on one kv head, head
# size 128, a window without blocks, four experts of sixteen, one looped layer, the loop's second pass starts inside the model.
F3 = {"architecture": "Fizelix", "vocab": 300, "width": 128, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.25}, "logit_scale": 3.0,
      "token_side": {"dim": 12}, "loop": {"start": 1, "stop": 2, "times": 2},
      "layers": [_attention(8, 1, 128, 32, 0.09, None, None, 64, 300000.0, _moe(16, 4, 32, 48)),
                 _attention(2, 2, 64, 64, 0.125, 500, 16, 32, 1000.0, _dense(64)),
                 _attention(4, 2, 32, 32, 0.2, 40, None, 8, 10000.0, None),
                 _mamba(2, 64, 16, 2, 4, 3, _dense(96))]}
CONFIGS = {"F1": F1, "F2": F2, "F3": F3}
LENGTHS = {"F1": [1, 2, 130, 61, 210, 37], "F2": [3, 75, 1, 140, 18, 66], "F3": [2, 90, 17, 1, 260, 40]}


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
        folder = os.path.join(str(tmp_path_factory.getbasetemp()), "fizelix_" + name)
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
    "tail": lambda r: H.trace_last_one_by_one(r, tail=100),     # long decoding: windows and blocks pass over decoded tokens
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


# ---- the comparison is sharp enough -------------------------------------------------------------------------------------
def _misread(monkeypatch, what):
    """One plausible misreading put into the plain implementation."""
    if what in ("window one token longer", "window one token shorter"):
        real = P.visible
        step = 1 if "longer" in what else -1
        monkeypatch.setattr(P, "visible", lambda i, window, block: real(i, window + step, block))
    elif what == "a block is seen as soon as it is complete":
        real = P.visible

        def early(i, window, block):
            tokens, _ = real(i, window, block)
            return tokens, ([b for b in range((i + 1) // block)] if block else [])
        monkeypatch.setattr(P, "visible", early)
    elif what == "a block is seen one token late":
        real = P.visible

        def late(i, window, block):
            tokens, _ = real(i, window, block)
            return tokens, real(i - 1, window, block)[1] if i > 0 else []
        monkeypatch.setattr(P, "visible", late)
    elif what == "no blocks":
        real = P.visible
        monkeypatch.setattr(P, "visible", lambda i, window, block: (real(i, window, block)[0], []))
    elif what == "weights normalised over the keys":
        def soft(h, W, p, heads, kv_heads, dim, vdim, scale, window, block, rot_dims, rot_base):
            T = h.shape[0]
            q = (h @ W[p + "q"].T).reshape(T, heads, dim)
            k = (h @ W[p + "k"].T).reshape(T, kv_heads, dim)
            v = (h @ W[p + "v"].T).reshape(T, kv_heads, vdim)
            if rot_dims:
                q, k = P.rotate_pairs(q, range(T), rot_dims, rot_base), P.rotate_pairs(k, range(T), rot_dims, rot_base)
            tok, _ = P.seen_masks(T, window, 0)
            out = [torch.softmax(((q[:, hd] @ k[:, hd // (heads // kv_heads)].T) * scale).masked_fill(~tok, -1e30), -1)
                   @ v[:, hd // (heads // kv_heads)] for hd in range(heads)]
            return torch.cat(out, -1) @ W[p + "o"].T
        monkeypatch.setattr(P, "pooled_sigmoid_attention", soft)
    elif what == "no bias per head":
        real = P.forward
        monkeypatch.setattr(P, "forward", lambda cfg, W, tokens, dtype=torch.float64, layers_out=None: real(
            cfg, {k: (torch.zeros_like(v) if k.endswith(".pb") else v) for k, v in W.items()}, tokens, dtype, layers_out))
    elif what == "halves rotated instead of adjacent pairs":
        def halves(x, positions, dims, base):
            out = x.clone()
            for i in range(dims // 2):
                a = torch.as_tensor([pos * base ** (-2.0 * i / dims) for pos in positions], dtype=x.dtype)[:, None]
                c, s = torch.cos(a), torch.sin(a)
                u, v = x[..., i], x[..., i + dims // 2]
                out[..., i], out[..., i + dims // 2] = u * c - v * s, v * c + u * s
            return out
        monkeypatch.setattr(P, "rotate_pairs", halves)
    elif what == "the expert's weight on its output":
        def on_output(h, W, p, experts, top, shared):
            s = torch.sigmoid(h @ W[p + "router"].T)
            out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=h.dtype)
            for t in range(h.shape[0]):
                for e in sorted(range(experts), key=lambda e: (-float(s[t, e]), e))[:top]:
                    out[t] = out[t] + s[t, e] * P.gated_unit(h[t][None], W, "%se%d." % (p, e))[0]
            return out + (P.gated_unit(h, W, p + "shared.") if shared else 0)
        monkeypatch.setattr(P, "routed_experts", on_output)
    elif what == "weights renormalised over the chosen experts":
        def renorm(h, W, p, experts, top, shared):
            s = torch.sigmoid(h @ W[p + "router"].T)
            out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=h.dtype)
            for t in range(h.shape[0]):
                chosen = sorted(range(experts), key=lambda e: (-float(s[t, e]), e))[:top]
                total = sum(s[t, e] for e in chosen)
                for e in chosen:
                    out[t] = out[t] + P.gated_unit((s[t, e] / total * h[t])[None], W, "%se%d." % (p, e))[0]
            return out + (P.gated_unit(h, W, p + "shared.") if shared else 0)
        monkeypatch.setattr(P, "routed_experts", renorm)
    elif what == "no shared expert":
        real = P.routed_experts
        monkeypatch.setattr(P, "routed_experts", lambda h, W, p, experts, top, shared: real(h, W, p, experts, top, False))
    elif what == "gate after the result's norm":
        def after(x, f, W, p, q, eps):
            h = P.unit_rms(x, eps) * W["%snorm%d" % (p, q)]
            y = P.unit_rms(f(h), eps) * W["%snorm%db" % (p, q)] * torch.sigmoid(h @ W["%srg%d" % (p, q)].T + W["%srg%d.b" % (p, q)])
            return x + y * W["%sls%d" % (p, q)]
        monkeypatch.setattr(P, "sublayer", after)
    elif what == "gate made from the stream, not from the sublayer's input":
        def from_stream(x, f, W, p, q, eps):
            h = P.unit_rms(x, eps) * W["%snorm%d" % (p, q)]
            y = f(h) * torch.sigmoid(x @ W["%srg%d" % (p, q)].T + W["%srg%d.b" % (p, q)])
            return x + P.unit_rms(y, eps) * W["%snorm%db" % (p, q)] * W["%sls%d" % (p, q)]
        monkeypatch.setattr(P, "sublayer", from_stream)
    elif what == "layer scale left out":
        real = P.forward
        monkeypatch.setattr(P, "forward", lambda cfg, W, tokens, dtype=torch.float64, layers_out=None: real(
            cfg, {k: (torch.ones_like(v) if k.endswith((".ls1", ".ls2")) else v) for k, v in W.items()}, tokens, dtype, layers_out))
    elif what == "the embedding joins every layer of a later pass":
        real = P.run_order

        def every(cfg):
            a = cfg["loop"]["start"]
            seen, out = set(), []
            for i, again in real(cfg):
                out.append((i, again or (i in seen and a <= i < cfg["loop"]["stop"])))
                seen.add(i)
            return out
        monkeypatch.setattr(P, "run_order", every)
    elif what == "the embedding never joins again":
        real = P.run_order
        monkeypatch.setattr(P, "run_order", lambda cfg: [(i, False) for i, _ in real(cfg)])
    elif what == "every layer reads the first layer's columns of the token table":
        real = P.token_side_input
        monkeypatch.setattr(P, "token_side_input", lambda x, tokens, W, p, index, dim, eps: real(x, tokens, W, p, 0, dim, eps))
    elif what == "the token input's gate made from the normed stream":
        def normed(x, tokens, W, p, index, dim, eps):
            e = W["side.embed"][torch.as_tensor(list(tokens), dtype=torch.long)][:, index * dim:(index + 1) * dim]
            g = P.gelu_tanh(P.unit_rms(x, eps) @ W[p + "side.gate"].T) * e
            return x + P.unit_rms(g @ W[p + "side.proj"].T, eps) * W[p + "side.norm"]
        monkeypatch.setattr(P, "token_side_input", normed)
    else:
        raise ValueError(what)


@pytest.mark.parametrize("what", [
    "window one token longer", "window one token shorter", "a block is seen as soon as it is complete", "a block is seen one token late",
    "no blocks", "weights normalised over the keys", "no bias per head", "halves rotated instead of adjacent pairs",
    "the expert's weight on its output", "weights renormalised over the chosen experts", "no shared expert",
    "gate after the result's norm", "gate made from the stream, not from the sublayer's input", "layer scale left out",
    "the embedding joins every layer of a later pass", "the embedding never joins again",
    "every layer reads the first layer's columns of the token table", "the token input's gate made from the normed stream"])
def test_a_misreading_of_the_design_shows(tmp_path_factory, monkeypatch, what):
    """The comparison the other tests rest on is sharp enough: with one misreading in the plain implementation the float32
    engine no longer agrees with it (the same request agrees without)."""
    folder, W = _model(tmp_path_factory, "F1")
    toks = H.random_tokens(F1["vocab"], 120, 21)
    engine = _engine(tmp_path_factory, "F1", torch.float32, 128)
    steps, _ = H.trace_whole({"a": toks})
    got = H.run_trace(engine, steps)
    H.compare(got, {"a": P.forward(F1, W, toks, torch.float64)}, 2e-4, "as designed")
    _misread(monkeypatch, what)
    with pytest.raises(AssertionError):
        H.compare(got, {"a": P.forward(F1, W, toks, torch.float64)}, 2e-4, what)


def test_the_residual_stream_after_every_layer(tmp_path_factory):
    """Layer by layer in float32, a looped layer counted each time: the stream after every entry of the run order."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "F1")
    toks = H.random_tokens(F1["vocab"], 45, 3)
    want = []
    P.forward(F1, W, toks, torch.float64, layers_out=want)
    eng = Engine.from_dir(folder, dtype=torch.float32, max_tokens=64, max_requests=1)
    got, build = [], eng._build_context

    def probed(entries, starts):
        ctx = build(entries, starts)
        ctx.layer_probe = lambda i, x, pending: got.append(x.clone())
        return ctx
    eng._build_context = probed
    eng.step([StepEntry("a", toks, [])])
    assert len(want) == 2 * 3 + 1 and len(got) == len(want) + 1
    for i, w in enumerate(want):
        assert torch.allclose(got[i].cpu().double(), w, atol=2e-5 * float(w.abs().max())), "after layer run %d" % i


@pytest.mark.parametrize("name,page_size", [("F1", 64), ("F3", 32)])
def test_other_page_sizes(tmp_path_factory, name, page_size):
    requests = _requests(name, seed=2)
    steps, max_tokens = H.trace_mixed(requests, seed=5)
    ref = _reference(tmp_path_factory, name, requests)
    engine = _engine(tmp_path_factory, name, torch.float32, max_tokens + 4 * page_size, page_size=page_size)
    H.compare(H.run_trace(engine, steps), ref, 2e-4, "%s page %d" % (name, page_size))
    engine.cache.check_invariants()


def test_recorded_decode_steps_equal_eager_ones(tmp_path_factory):
    """Long decoding past the window and over many blocks: the same request decoded through recorded steps and eagerly
    gives the same logits; states and block means move on exactly once per step, also in the step that is recorded."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "F1")
    toks = H.random_tokens(F1["vocab"], 200, 9)
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
    ref = P.forward(F1, W, toks, torch.float64)[30:]
    assert float((rows[True].double() - ref).abs().max()) <= 2e-4 * float(ref.abs().max())


def test_a_forked_request_goes_on_apart(tmp_path_factory):
    """A copy of a request (its pages of both kinds and its states) and the original continue with different tokens."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "F1")
    toks = H.random_tokens(F1["vocab"], 70, 11)
    a_tail, b_tail = H.random_tokens(F1["vocab"], 30, 12), H.random_tokens(F1["vocab"], 30, 13)
    eng = Engine.from_dir(folder, dtype=torch.float32, max_tokens=512, page_size=16, max_requests=3, use_graphs=False)
    eng.step([StepEntry("a", toks, [])])
    eng.fork("a", "b")
    la = eng.step([StepEntry("a", a_tail, list(range(30)))]).float().cpu().clone()
    lb = eng.step([StepEntry("b", b_tail, list(range(30)))]).float().cpu().clone()
    for got, tail in ((la, a_tail), (lb, b_tail)):
        ref = P.forward(F1, W, toks + tail, torch.float64)[70:]
        assert float((got.double() - ref).abs().max()) <= 2e-4 * float(ref.abs().max())
    eng.free("a")
    eng.free("b")
    eng.cache.check_invariants()


# ---- each mechanism's kernel alone ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,G,dk,dv,rot,base,extra", [(6, 3, 24, 40, 10, 77.0, 13), (4, 2, 64, 32, 64, 10000.0, 0), (3, 1, 128, 8, 32, 300000.0, 24),
                                                       (2, 2, 16, 16, 0, None, 8)])
def test_rotation_of_adjacent_pairs_with_the_cache_write(dtype, Hq, G, dk, dv, rot, base, extra):
    """The first ``rot`` entries of every query and key head turn in pairs (2i, 2i+1), the rest pass; positions up to
    60,000 keep float32 accuracy; keys and values land in their pages."""
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.parts.pooled_attention import pair_frequencies
    page = 16
    positions = [0, 1, 2, 17, 1000, 4095, 59999, 60000, 33]
    T = len(positions)
    g = torch.Generator().manual_seed(dk + rot)
    n = (Hq + G) * dk + G * dv
    rows = (2 * torch.randn(T, n + extra, generator=g)).to(dtype)
    kc = torch.zeros(4, G, page, dk, dtype=dtype, device="cuda")
    vc = torch.zeros(4, G, page, dv, dtype=dtype, device="cuda")
    slots = [33, 34, 35, 2, 47, 48, 16, 0, 63]
    q_out = torch.empty(T, Hq * dk, dtype=dtype, device="cuda")
    freq = pair_frequencies(rot, base).cuda() if rot else None
    ops.rope_pairs_store(_dev(rows), _i32(positions), freq, rot, q_out, kc, vc, _i32(slots), Hq, G, dk, dv, page)
    full = rows[:, :n].double()
    q, k = full[:, :Hq * dk].view(T, Hq, dk), full[:, Hq * dk:(Hq + G) * dk].view(T, G, dk)
    if rot:
        q, k = P.rotate_pairs(q, positions, rot, base), P.rotate_pairs(k, positions, rot, base)
    v = full[:, (Hq + G) * dk:].view(T, G, dv)
    tol = 2e-6 * float(full.abs().max()) if dtype == torch.float32 else 3e-2
    assert torch.allclose(q_out.cpu().double(), q.reshape(T, -1), atol=tol)
    for t, s in enumerate(slots):
        assert torch.allclose(kc[s // page, :, s % page].cpu().double(), k[t], atol=tol)
        assert torch.equal(vc[s // page, :, s % page].cpu().double(), v[t])


class _Paged:
    """Keys and values of several requests laid out in shuffled pages, with the means of their complete blocks in shuffled
    pages of their own; unused pages hold NaN."""

    def __init__(self, lens, G, dk, dv, page, block, dtype, seed, extra_pages=3):
        g = torch.Generator().manual_seed(seed)
        self.k = [torch.randn(n, G, dk, generator=g).to(dtype) for n in lens]
        self.v = [torch.randn(n, G, dv, generator=g).to(dtype) for n in lens]
        self.kc, self.vc, self.bt = self._lay(self.k, self.v, page, seed, extra_pages)
        if block:
            self.km = [k[:len(k) // block * block].double().view(-1, block, G, dk).mean(1).to(dtype) for k in self.k]
            self.vm = [v[:len(v) // block * block].double().view(-1, block, G, dv).mean(1).to(dtype) for v in self.v]
            self.kp, self.vp, self.pt = self._lay(self.km, self.vm, page, seed + 1, extra_pages)

    @staticmethod
    def _lay(ks, vs, page, seed, extra_pages):
        lens = [len(k) for k in ks]
        G, dk, dv, dtype = ks[0].shape[1], ks[0].shape[2], vs[0].shape[2], ks[0].dtype
        need = [(n + page - 1) // page for n in lens]
        ids = list(range(sum(need) + extra_pages))
        random.Random(seed).shuffle(ids)
        kc = torch.full((len(ids), G, page, dk), float("nan")).to(dtype)
        vc = torch.full((len(ids), G, page, dv), float("nan")).to(dtype)
        bt = torch.zeros(len(lens), max(need + [1]), dtype=torch.int32)
        bt[:] = ids[-1]                                        # entries past a request's pages point at a NaN page
        for r, n in enumerate(lens):
            for j in range(need[r]):
                pg = ids.pop(0)
                bt[r, j] = pg
                lo, hi = j * page, min(n, (j + 1) * page)
                kc[pg, :, :hi - lo] = ks[r][lo:hi].transpose(0, 1)
                vc[pg, :, :hi - lo] = vs[r][lo:hi].transpose(0, 1)
                kc[pg, :, hi - lo:] = 0                        # the rest of a request's last page: written later, finite
                vc[pg, :, hi - lo:] = 0
        return kc, vc, bt


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("G,dk,dv,block,page", [(2, 32, 64, 8, 16), (3, 10, 12, 1, 16), (1, 128, 128, 20, 32), (2, 24, 8, 5, 16), (1, 64, 64, 64, 16)])
def test_means_of_the_blocks_a_step_completes(dtype, G, dk, dv, block, page):
    """Portions that end a block with their first token, in their middle, with their last token or not at all, several
    blocks in one portion, single tokens: exactly the completed blocks' rows are written, as means of what the cache holds."""
    from infinicore_infer_amd.kernels import ops
    lens = [150, 70, 9]
    pg = _Paged(lens, G, dk, dv, page, block, dtype, seed=dk + block)
    kc, vc, bt, pt = pg.kc.cuda(), pg.vc.cuda(), pg.bt.cuda(), pg.pt.cuda()
    kp = torch.full(pg.kp.shape, float("nan")).to(dtype).cuda()
    vp = torch.full(pg.vp.shape, float("nan")).to(dtype).cuda()
    steps = [[(0, 0, 150), (1, 0, 3), (2, 0, 1)], [(1, 3, block), (2, 1, 2)], [(1, 3 + block, 1)], [(1, 4 + block, 70 - 4 - block), (2, 3, 6)]]
    done = {0: 0, 1: 0, 2: 0}
    for step in steps:
        positions = sum((list(range(p0, p0 + n)) for r, p0, n in step), [])
        req_rows = [0]
        for _, _, n in step:
            req_rows.append(req_rows[-1] + n)
        rows = torch.tensor([r for r, _, _ in step])
        ops.pool_blocks(kc, vc, kp, vp, bt[rows].contiguous(), pt[rows].contiguous(), _i32(req_rows), _i32(positions), len(step),
                        max(n for _, _, n in step), block, G, dk, dv, page)
        for r, p0, n in step:
            done[r] = (p0 + n) // block
        for r in range(3):
            for b in range(len(pg.km[r])):
                got = kp[pt[r, b // page].item(), :, b % page].float().cpu()
                if b < done[r]:
                    tol = 1e-6 if dtype == torch.float32 else 1e-2
                    assert torch.allclose(got.double(), pg.km[r][b].double(), atol=tol), (r, b)
                    assert torch.allclose(vp[pt[r, b // page].item(), :, b % page].float().cpu().double(), pg.vm[r][b].double(), atol=tol), (r, b)
                else:
                    assert torch.isnan(got).all(), "block %d of request %d written before it was complete" % (b, r)


ATTENTION_CASES = [
    # heads, kv heads, dk, dv, window, block, page
    (4, 2, 64, 32, 36, 12, 16),
    (4, 2, 32, 64, 64, 8, 16),
    (8, 1, 128, 128, 100, 32, 32),
    (2, 2, 64, 64, 0, 0, 64),
    (6, 3, 128, 32, 31, 5, 16),
    (3, 1, 24, 40, 17, 20, 16),
    (2, 1, 16, 16, 1, 1, 16),
    (2, 2, 32, 32, 48, 0, 16),
    (6, 2, 64, 128, 20, 4, 16),            # three query heads a kv head; (10, 2, ..): five, two walks of the single tokens' kernel
    (10, 2, 128, 64, 70, 7, 32),
]


@pytest.mark.parametrize("dname,dtype,tol", [("float32", torch.float32, 2e-5), ("bfloat16", torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("case", ATTENTION_CASES)
def test_attention_over_a_window_and_block_means(case, dname, dtype, tol):
    """The attention kernels against dense sigmoid weights under the plain masks: prompt portions that start anywhere,
    single tokens at, just before and just after every edge (the window's, a block's, a page's, a 64-item step's), with one
    token's score made to stand out just inside and just outside the window and one block's just seen and not yet seen;
    pages shuffled, NaN in every page a kernel must not read (also in the rows of blocks that are not yet complete)."""
    from infinicore_infer_amd.kernels import ops
    H_, G, dk, dv, window, block, page = case
    scale = 1.7 / math.sqrt(dk)
    lens = [300, 150, 7]
    pg = _Paged(lens, G, dk, dv, page, block, dtype, seed=dk + dv + window)
    g = torch.Generator().manual_seed(7)
    kc, vc, bt = pg.kc.cuda(), pg.vc.cuda(), pg.bt.cuda()
    kp, vp, pt = (pg.kp.cuda(), pg.vp.cuda(), pg.pt.cuda()) if block else (None, None, None)
    bias = torch.tensor(([-2.0, 0.5, -4.0, 1.0] * 3)[:H_])

    def run(kernel, req_rows):
        qs, refs, token_req, positions, tiles, row = [], [], [], [], [], 0
        for r, p0, n in req_rows:
            q = torch.randn(n, H_ * dk, generator=g)
            last = p0 + n - 1
            if window:       # the last query leans on the token just inside / just outside the window, or on the newest / the next block
                rnd = random.Random(last + n)
                for target in (last - window + 1, last - window):
                    if 0 <= target and rnd.random() < 0.6:
                        q[n - 1].view(H_, dk)[:] += 6.0 * pg.k[r][target].float().repeat_interleave(H_ // G, 0)
                if block:
                    nb = max(0, last - window + 1) // block
                    for b in (nb - 1, nb):
                        if 0 <= b < len(pg.km[r]) and rnd.random() < 0.6:
                            q[n - 1].view(H_, dk)[:] += 6.0 * block * pg.km[r][b].float().repeat_interleave(H_ // G, 0)
            q = q.to(dtype)
            T = p0 + n
            tok, blk = P.seen_masks(n, window or None, block, first=p0)
            out = []
            for h in range(H_):
                gi = h // (H_ // G)
                qh = q.double().view(n, H_, dk)[:, h]
                o = (torch.sigmoid((qh @ pg.k[r][:T, gi].double().T) * scale + bias[h].double()) * tok) @ pg.v[r][:T, gi].double()
                if blk.shape[1]:
                    nb = blk.shape[1]
                    o = o + (torch.sigmoid((qh @ pg.km[r][:nb, gi].double().T) * scale + bias[h].double()) * blk) @ pg.vm[r][:nb, gi].double()
                out.append(o)
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
        args = (kc, vc, kp, vp, bt, pt)
        tail = (bias.cuda(), H_, G, dk, dv, page, scale, window, block)
        if kernel == "general":
            ops.attention_pooled_generic(q, out, *args, tr, ps_, *tail)
        elif kernel == "prefill":
            ops.attention_pooled_prefill(q, out, *args, _i32(sum(map(list, tiles), [])), len(tiles), *tail)
        else:
            ns = int(kernel)
            parts = torch.full((ns * row * H_ * dv,), float("nan"), dtype=torch.float32, device="cuda")
            ops.attention_pooled_decode(q, out, *args, None, row, tr, ps_, parts, *tail, n_split=ns)
        ref = torch.cat(refs)
        err = float((out.float().cpu().double() - ref).abs().max()) / max(1.0, float(ref.abs().max()))
        assert math.isfinite(err) and err <= tol, "%s: error %.3g (allowed %.3g)" % (kernel, err, tol)

    edges = sorted({0, 1, window - 2, window - 1, window, window + 1, window + block - 2, window + block - 1, window + block,
                    window + 2 * block - 1, page - 1, page, 63, 64, 65, 127, 128, 149, 299} - {-1, -2})
    singles = [(0, p, 1) for p in edges if p < 300] + [(1, p, 1) for p in edges if p < 150] + [(2, 6, 1)]
    portions = [(0, 0, 300), (1, 0, 2), (2, 0, 7), (1, 2, 131), (0, 171, 129), (1, 133, 17), (0, 64, 2), (0, 40, 70)]
    run("general", singles + portions)
    if ops.attention_pooled_decode_supported(dtype, dk, dv):
        for ns in (1, 2, 7):
            run(str(ns), singles)
    if ops.attention_pooled_prefill_supported(dtype, dk, dv, page):
        run("prefill", portions + singles[:5])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,top,d,ff,mode,renorm,on_input", [(5, 4, 2, 32, 24, "sigmoid", False, True), (70, 3, 1, 70, 30, "sigmoid", False, True),
                                                                (9, 16, 4, 64, 40, "softmax", True, False), (1, 2, 2, 128, 96, "sigmoid", True, True),
                                                                (33, 5, 3, 20, 12, "softmax", False, False), (6, 8, 2, 2304, 64, "sigmoid", False, True)])
def test_routed_experts_kernels(dtype, T, E, top, d, ff, mode, renorm, on_input):
    """Choice and weights (ties go to the lower index), the stable sort by expert, the gathered and weighted rows, both
    products of every expert's rows with the gated unit between them, and the sum per token with a shared row."""
    from infinicore_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(T + E)
    z = 2 * torch.randn(T, E, generator=g)
    z[0, :] = 0.25                                             # a tie among all experts
    if T > 2:
        z[2, -1] = z[2, 0]
    ids = torch.empty(T, top, dtype=torch.int32, device="cuda")
    w = torch.empty(T, top, dtype=torch.float32, device="cuda")
    ops.moe_route(z.cuda(), top, ids, w, mode, renorm)
    s = torch.sigmoid(z.double()) if mode == "sigmoid" else torch.softmax(z.double(), -1)
    want_ids = [sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top] for t in range(T)]
    assert ids.cpu().tolist() == want_ids
    want_w = torch.stack([s[t, want_ids[t]] for t in range(T)])
    if renorm:
        want_w = want_w / want_w.sum(-1, keepdim=True)
    assert torch.allclose(w.cpu().double(), want_w, atol=1e-6)
    n = T * top
    offsets, order, place = (torch.empty(m, dtype=torch.int32, device="cuda") for m in (E + 1, n, n))
    ops.moe_sort(ids, E, offsets, order, place)
    flat = [e for row in want_ids for e in row]
    want_order = sorted(range(n), key=lambda i: (flat[i], i))
    assert order.cpu().tolist() == want_order
    assert offsets.cpu().tolist() == [sum(e < b for e in flat) for b in range(E + 1)]
    assert [order.cpu().tolist()[p] for p in place.cpu().tolist()] == list(range(n))
    h = torch.randn(T, d + 8, generator=g).to(dtype)[:, :d]
    rows = torch.empty(n, d, dtype=dtype, device="cuda")
    ops.moe_gather(h.cuda(), order, w.view(-1) if on_input else None, top, rows)
    want_rows = torch.stack([h[i // top].double() * (want_w.view(-1)[i] if on_input else 1.0) for i in want_order])
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert torch.allclose(rows.cpu().double(), want_rows, atol=tol * float(h.abs().max()))
    wgu = (torch.randn(E, 2 * ff, d, generator=g) / math.sqrt(d)).to(dtype)
    wdn = (torch.randn(E, d, ff, generator=g) / math.sqrt(ff)).to(dtype)
    act = torch.empty(n, ff, dtype=dtype, device="cuda")
    y = torch.empty(n, d, dtype=dtype, device="cuda")
    ops.moe_expert_product(rows, wgu.cuda(), offsets, act, glu=True)
    ops.moe_expert_product(act, wdn.cuda(), offsets, y, glu=False)
    rr = rows.cpu().double()
    want_act = torch.stack([P.silu(rr[j] @ wgu[flat[i], :ff].double().T) * (rr[j] @ wgu[flat[i], ff:].double().T) for j, i in enumerate(want_order)])
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(act.cpu().double(), want_act, atol=tol * max(1.0, float(want_act.abs().max())))
    aa = act.cpu().double()
    want_y = torch.stack([aa[j] @ wdn[flat[i]].double().T for j, i in enumerate(want_order)])
    assert torch.allclose(y.cpu().double(), want_y, atol=tol * max(1.0, float(want_y.abs().max())))
    shared = torch.randn(T, d, generator=g).to(dtype)
    out = torch.empty(T, d, dtype=dtype, device="cuda")
    ops.moe_combine(y, place, None if on_input else w.view(-1), shared.cuda(), top, out)
    yy, pl = y.cpu().double(), place.cpu().tolist()
    want_out = torch.stack([shared[t].double() + sum(yy[pl[t * top + k]] * (1.0 if on_input else want_w[t, k]) for k in range(top)) for t in range(T)])
    assert torch.allclose(out.cpu().double(), want_out, atol=tol * max(1.0, float(want_out.abs().max())))


@pytest.mark.parametrize("d,ff", [(48, 40), (64, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_experts_part_for_few_and_many_rows(dtype, d, ff):
    """The part with few rows (no integer leaves the device; sizes the matrix-core product takes and sizes it does not, more
    than sixteen rows an expert) and with many (one library product per expert) against the plain feed-forward; the weight on
    the expert's input, a shared expert, four experts of six."""
    from infinicore_infer_amd.engine.context import StepContext, Workspace
    from infinicore_infer_amd.parts import Runtime
    from infinicore_infer_amd.parts.routed_experts import RoutedExperts
    E, top, sh = 6, 4, 56
    cfg = {"vocab": 8, "width": d, "layers": [{"type": "attention", "mixer": {"heads": 1, "dim": 8}, "mlp": _moe(E, top, ff, sh)}]}
    W = {k[len("l0.mlp."):]: v for k, v in P.random_weights(cfg, 5).items() if k.startswith("l0.mlp.")}
    part = RoutedExperts("", Runtime(dtype, "cuda"), d, E, top, ff, sh)
    tensors = {k: v.to(dtype).cuda() for k, v in W.items()}
    part.load_weights(tensors)
    part.shared.load_weights(tensors)
    ctx = StepContext()
    ctx.ws, ctx.cu_count = Workspace("cuda"), 256
    g = torch.Generator().manual_seed(3)
    for T in (1, 7, 64, 65, 300):
        h = torch.randn(T, d, generator=g).to(dtype)
        got = part.forward(h.cuda(), ctx).float().cpu().double()
        want = P.routed_experts(h.double(), {k: v.double() for k, v in W.items()}, "", E, top, True)
        if dtype == torch.float32:
            assert torch.allclose(got, want, atol=2e-5 * float(want.abs().max())), T
        else:
            err = (got - want).abs().amax(-1) / float(want.abs().max())
            assert float(err.mean()) < 1e-2 and int((err > 5e-2).sum()) <= max(1, T // 30), (T, float(err.max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,d", [(5, 70), (3, 256), (2, 2304)])
def test_gate_on_a_result_and_its_norm_into_the_stream(dtype, T, d):
    from infinicore_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(d)
    y, gate = (3 * torch.randn(T, d, generator=g)).to(dtype), (2 * torch.randn(T, d + 8, generator=g)).to(dtype)[:, :d]
    gb, w, x, eps = torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g), torch.randn(T, d, generator=g), 1e-5
    for use_gate in (True, False):
        xs = x.clone().cuda()
        copy = torch.empty(T, d, dtype=dtype, device="cuda")
        ops.gated_norm_into_stream(y.cuda(), gate.cuda() if use_gate else None, gb.cuda() if use_gate else None, w.cuda(), xs, eps, copy=copy)
        v = y.double() * (torch.sigmoid(gate.double() + gb.double()) if use_gate else 1.0)
        want = x.double() + P.unit_rms(v, eps) * w.double()
        assert torch.allclose(xs.cpu().double(), want, atol=1e-5)
        assert torch.allclose(copy.float().cpu().double(), want, atol=1e-5 if dtype == torch.float32 else 5e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_on_a_slice_of_a_token_table(dtype):
    from infinicore_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    T, n, width, vocab = 7, 12, 40, 30
    z = (3 * torch.randn(T, n + 4, generator=g)).to(dtype)[:, :n]
    table = torch.randn(vocab, width, generator=g).to(dtype)
    tokens = [3, 29, 0, 3, 17, 8, 1]
    out = torch.empty(T, n, dtype=dtype, device="cuda")
    ops.token_gate(z.cuda(), table.cuda(), _i32(tokens), 24, out)
    want = P.gelu_tanh(z.double()) * table.double()[tokens][:, 24:36]
    assert torch.allclose(out.float().cpu().double(), want, atol=1e-5 if dtype == torch.float32 else 5e-2)


# ---- generation through the entry point --------------------------------------------------------------------------------
def _plain_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(P.forward(cfg, W, toks, torch.float64)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["F1", "F2", "F3"])
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
    folder, W = _model(tmp_path_factory, "F2")
    prompt = H.random_tokens(F2["vocab"], 9, 77)
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.fizelix", "--amd", folder, "--dtype", "float32",
                        "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--max-tokens", "128"],
                       cwd=H.__file__.rsplit("/tests/", 1)[0], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    want = _plain_greedy(F2, W, prompt, 6)
    assert " ".join(map(str, want)) in " ".join(r.stdout.split()), r.stdout[-2000:]


def test_command_line_with_random_weights(tmp_path):
    import subprocess
    import sys
    path = str(tmp_path / "config.json")
    with open(path, "w") as f:
        json.dump(F3, f)
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
    folder, W = _model(tmp_path_factory, "F2")
    requests = _requests("F2", seed=4)
    steps, max_tokens = H.trace_mixed(requests, seed=3)
    root = H.__file__.rsplit("/tests/", 1)[0]
    out = str(tmp_path / "out")
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out,
                        "--max-tokens", str(max_tokens)], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.split("\n") if l.startswith("done")] == ["done %d" % s["step"] for s in steps]
    ref = {rid: P.forward(F2, W, toks, torch.float64) for rid, toks in requests.items()}
    at, got = {}, {}
    for s in steps:
        rows = torch.frombuffer(bytearray(open(os.path.join(out, "%d.f32" % s["step"]), "rb").read()), dtype=torch.float32).view(-1, F2["vocab"])
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

    def mlp():
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return _dense(rng.choice([24, 50, 128]))
        experts = rng.choice([2, 3, 8, 11])
        return _moe(experts, rng.randint(1, min(experts, 4)), rng.choice([12, 30, 64]), rng.choice([None, 20, 64]))
    for _ in range(rng.choice([2, 3, 4])):
        if rng.random() < 0.35:
            groups = rng.choice([1, 2, 3])
            heads = groups * rng.choice([1, 2])
            vdim = rng.choice([8, 12, 32])
            ng = rng.choice([g for g in (1, 2, 3, 4, 6) if (heads * vdim) % g == 0 and heads * vdim // g >= 8])
            layers.append(_mamba(heads, vdim, rng.choice([4, 9, 16, 40]), groups, ng, rng.choice([1, 2, 3, 4]), mlp()))
        else:
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([8, 12, 32, 64])
            window = rng.choice([None, 1, 2, 15, 16, 33, 100])
            pool = rng.choice([None, 1, 3, 16, 40]) if window else None
            rot = rng.choice([0, 2, dim // 2, dim])
            rot -= rot % 2
            layers.append(_attention(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([4, 20, 32, 64]), round(rng.uniform(0.05, 0.4), 3),
                                     window, pool, rot, rng.choice([100.0, 10000.0, 300000.0]), mlp()))
    cfg = {"architecture": "Fizelix", "vocab": rng.choice([53, 128, 301]), "width": width, "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])},
           "embedding": {"scale": rng.choice([1.0, 0.5, 4.0])}, "logit_scale": rng.choice([1.0, 2.0, 0.3]), "layers": layers}
    if rng.random() < 0.7:
        a = rng.randrange(len(layers))
        cfg["loop"] = {"start": a, "stop": rng.randint(a, len(layers)), "times": rng.choice([1, 2, 3])}
    if rng.random() < 0.7:
        cfg["token_side"] = {"dim": rng.choice([1, 5, 16])}
    return cfg


@pytest.mark.parametrize("seed", list(range(12)))
def test_drawn_configurations(tmp_path_factory, seed):
    from infinicore_infer_amd.engine import Engine
    cfg = _drawn_config(seed)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "fizelix_drawn_%d" % seed)
    W = _write_model(folder, cfg, seed)
    rng = random.Random(seed + 100)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab"], n, seed * 10 + i)
                for i, n in enumerate([rng.choice([1, 2, 5, 40, 66, 129, 150]) for _ in range(5)])}
    ref = {rid: P.forward(cfg, W, toks, torch.float64) for rid, toks in requests.items()}
    steps, max_tokens = H.trace_mixed(requests, seed=seed)
    for dname, dtype, tol in DTYPES:
        engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=16, max_requests=4)
        _compare(H.run_trace(engine, steps), ref, dtype, tol if dtype == torch.float32 else 0.3, "drawn %d %s" % (seed, dname), steps, loose=True)
        engine.cache.check_invariants()
        assert not engine.cache.requests
