"""Host-side parts of the Fizelix decoder: its configuration and its errors, the run order of a looped stretch, the model
as data, what its parts ask of the cache manager (rows per token in a window group, rows per block of tokens in a
group of their own), weights loaded into fused layouts, and the plain implementation's own properties."""
import json
import math
import random

import pytest
import torch

import plain_fizelix as P
from test_gpu_fizelix import F1, F2, F3, _write_model

from infinicore_infer_amd.cache import CacheError, CacheManager, GroupSpec, OutOfPages
from infinicore_infer_amd.config import ConfigError, config_from_dict
from infinicore_infer_amd.parts import Runtime, build_model


def test_config_to_model_spec():
    cfg = config_from_dict(F1)
    spec = cfg.model_spec()
    assert spec.architecture == "Fizelix" and spec.vocab_size == 211 and spec.hidden_size == 96 and spec.residual_streams == 1
    # layers 0..1 three times in a row, every pass with cache slots of its own; the embedding joins before passes two and three
    assert [(e.layer, e.cache, e.adds_embedding) for e in spec.schedule] == [
        (0, 0, False), (1, 1, False), (0, 2, True), (1, 3, False), (0, 4, True), (1, 5, False), (2, 6, False)]
    assert [l.mixer.kind for l in spec.layers] == ["pooled_attention", "mamba2", "pooled_attention"]
    assert all(l.block.kind == "sandwich_gated" for l in spec.layers)
    a = spec.layers[0].mixer.params
    assert (a["num_heads"], a["num_kv_heads"], a["key_dim"], a["value_dim"], a["window"], a["block"]) == (4, 2, 32, 64, 24, 8)
    assert (a["rot_dims"], a["rot_base"], a["score_scale"], a["weights"], a["head_bias"]) == (16, 10000.0, 0.18, "sigmoid", True)
    b = spec.layers[0].block.params
    assert (b["mixer_out_norm"].params["tensor"], b["mixer_out_norm"].params["scale_tensor"]) == ("l0.norm1b", "l0.ls1")
    assert (b["feed_forward_out_norm"].params["tensor"], b["feed_forward_out_norm"].params["scale_tensor"]) == ("l0.norm2b", "l0.ls2")
    assert b["gated"] and (b["side"]["first_column"], b["side"]["dim"], b["side"]["table_width"]) == (0, 8, 24)
    assert spec.layers[2].block.params["side"]["first_column"] == 16 and spec.layers[2].block.params["side"]["norm"].params["tensor"] == "l2.side.norm"
    assert spec.layers[0].mixer_norm.params["tensor"] == "l0.norm1" and spec.layers[0].mixer_norm.params["scale_tensor"] is None
    f = spec.layers[1].feed_forward
    assert f.kind == "routed_experts" and (f.params["experts"], f.params["top"], f.params["expert_size"], f.params["shared_size"]) == (4, 2, 48, 64)
    assert (f.params["scores"], f.params["renormalize"], f.params["weight_on"]) == ("sigmoid", False, "input")
    assert spec.layers[2].feed_forward.params["shared_size"] is None and spec.layers[0].feed_forward.kind == "swiglu"
    assert (spec.embedding.params["scale"], spec.head.params["logit_scale"]) == (3.0, 0.5)
    assert config_from_dict(cfg.to_dict()).model_spec().layers[0].mixer.params == a
    assert config_from_dict(F1, max_tokens=300).max_positions == 300 and cfg.context_is_open
    # no loop, no token input, no mask, no rotation, a layer without a feed-forward
    plain = config_from_dict(F2).model_spec()
    assert [(e.layer, e.adds_embedding) for e in plain.schedule] == [(0, False), (1, False), (2, False)]
    assert plain.layers[0].block.params["side"] is None and plain.layers[1].feed_forward is None
    assert plain.layers[1].block.params["feed_forward_out_norm"] is None and plain.layers[2].mixer.params["rot_dims"] == 0
    assert (plain.embedding.params["scale"], plain.head.params["logit_scale"]) == (1.0, 1.0)
    inside = config_from_dict(F3)
    assert [(e.layer, e.adds_embedding) for e in inside.model_spec().schedule] == [(0, False), (1, False), (1, True), (2, False), (3, False)]
    assert inside.model_spec().layers[0].mixer.params["window"] is None and inside.model_spec().layers[0].mixer.params["block"] is None
    assert inside.model_spec().layers[2].mixer.params["block"] is None
    # an empty loop, and a loop of one pass, change nothing
    for loop in ({"start": 1, "stop": 1, "times": 5}, {"start": 0, "stop": 3, "times": 1}):
        c = config_from_dict(dict(F1, loop=loop))
        assert c.run_order() == [(0, False), (1, False), (2, False)]


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="lightning"), "type"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].pop("norm_groups"), "norm_groups"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "dense or moe"),
    (lambda c: c["layers"][1]["mlp"].pop("router"), "router"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("ff"), "ff"),
    (lambda c: c.update(layers=[]), "layers"),
    (lambda c: c["loop"].update(stop=7), "loop"),
    (lambda c: c["loop"].pop("times"), "times"),
    (lambda c: c["token_side"].update(dim=-2), "token_side"),
])
def test_config_errors(change, what):
    cfg = json.loads(json.dumps(F1))
    change(cfg)
    with pytest.raises(ConfigError) as e:
        config_from_dict(cfg)
    assert what in str(e.value)


def test_part_errors():
    from infinicore_infer_amd.parts.base import build_part, CacheNeed
    from infinicore_infer_amd.config import PartSpec
    rt = Runtime(torch.float32, "cpu")
    att = {"hidden_size": 16, "num_heads": 2, "num_kv_heads": 1, "key_dim": 8, "value_dim": 8, "score_scale": 0.3}
    for bad in ({"num_kv_heads": 3}, {"rot_dims": 6, "rot_base": None}, {"rot_dims": 5, "rot_base": 10.0}, {"rot_dims": 10, "rot_base": 10.0},
                {"weights": "softmax"}, {"key_dim": 600}):
        with pytest.raises(ValueError):
            build_part("mixer", PartSpec("pooled_attention", "a.", dict(att, **bad)), rt)
    moe = {"hidden_size": 16, "experts": 4, "top": 2, "expert_size": 8}
    for bad in ({"top": 5}, {"top": 0}, {"scores": "tanh"}, {"weight_on": "both"}, {"expert_size": 0}):
        with pytest.raises(ValueError):
            build_part("feed_forward", PartSpec("routed_experts", "f.", dict(moe, **bad)), rt)
    with pytest.raises(ValueError):
        CacheNeed("state", state_shape=(4,), block_rows=8)
    with pytest.raises(CacheError):
        GroupSpec("window", 1, 8, 16, (0,), stride=4, of_blocks=True)


def test_cache_needs_of_the_mixers():
    model = build_model(config_from_dict(F1).model_spec(), Runtime(torch.float32, "cpu"))
    needs = model.cache_needs()
    assert [n.kind for n in needs] == ["kv", "state", "kv", "state", "kv", "state", "kv"]
    att, ssm, last = needs[0], needs[1], needs[6]
    assert (att.planes, att.n_kv_heads, att.plane_dims, att.window, att.block_rows) == (2, 2, (32, 64), 24, 8)
    # the token cache keeps as many tokens as the longer of window and block: a block's tokens are there when it is complete
    assert (last.window, last.block_rows) == (33, 5)
    model2 = build_model(config_from_dict(F2).model_spec(), Runtime(torch.float32, "cpu"))
    assert [(n.window, n.block_rows) for n in model2.cache_needs() if n.paged] == [(1, 1), (20, 20)]
    model3 = build_model(config_from_dict(F3).model_spec(), Runtime(torch.float32, "cpu"))
    assert [(n.window, n.block_rows) for n in model3.cache_needs() if n.paged] == [(None, 0), (500, 16), (500, 16), (40, 0)]
    assert ssm.state_shape == (4 * 24 * 16 + 3 * (64 + 2 * 2 * 24),) and needs[2] == att and needs[3] == ssm


def test_rows_per_block_of_tokens_in_the_cache_manager():
    """A strided group holds one row for every complete block of tokens: its pages come when a block is complete, go back
    only with the request, follow a truncation, and a fork copies exactly the pages that hold complete blocks."""
    page, stride = 4, 3
    groups = [GroupSpec("window", 1, 8, 6, (0,)), GroupSpec("full", 1, 8, None, (0,), stride=stride, of_blocks=True)]
    cm = CacheManager(groups, [8, 3], page, 3)
    cm.admit("a")
    assert cm.pages_for_tokens(0) == [0, 0] and cm.pages_for_tokens(2) == [1, 0] and cm.pages_for_tokens(3) == [1, 1]
    assert cm.pages_for_tokens(14) == [4, 1] and cm.pages_for_tokens(15) == [4, 2]
    cm.append("a", 2)
    assert [len(t) for t in cm.requests["a"].tables] == [1, 0]
    assert cm.pages_needed("a", 1) == [0, 1]              # the third token completes block 0
    cm.append("a", 1)
    assert [len(t) for t in cm.requests["a"].tables] == [1, 1]
    cm.append("a", 11)                                    # 14 tokens: four complete blocks, one page
    assert [len(t) for t in cm.requests["a"].tables] == [4, 1]
    cm.trim("a")                                          # the window group gives back what lies before the window
    assert cm.requests["a"].tables[0][:2] == [-1, -1] and cm.requests["a"].tables[1][0] >= 0
    assert cm.pages_needed("a", 1) == [0, 1]              # the fifth block needs the second page
    cm.append("a", 1)
    cm.check_invariants()
    cm.truncate("a", 14)
    assert [len(t) for t in cm.requests["a"].tables] == [4, 1]
    slot, pairs = cm.fork("a", "b")
    assert sorted(g for g, _, _ in pairs) == [0, 0, 1] and [len(t) for t in cm.requests["b"].tables] == [4, 1]
    cm.admit("c")
    cm.append("c", 12)                                    # blocks 0..3 of c: one page; b and a hold one each
    with pytest.raises(OutOfPages):
        cm.append("c", 20)                                # 32 tokens: ten blocks, three pages; the pool of three has none left
    assert cm.length("c") == 12
    cm.check_invariants()
    for r in ("a", "b", "c"):
        cm.release(r)
    assert cm.free_pages(0) == 8 and cm.free_pages(1) == 3
    # random orders of growth, trimming and release keep every page accounted for
    rng = random.Random(1)
    live = {}
    for _ in range(300):
        r = rng.randrange(3)
        if r not in live and cm.can_admit():
            cm.admit(r)
            live[r] = 0
        elif r in live and rng.random() < 0.2:
            cm.release(r)
            del live[r]
        elif r in live:
            n = rng.choice([1, 1, 2, 5])
            if cm.can_append(r, n):
                cm.append(r, n)
                live[r] += n
                cm.trim(r)
                assert len(cm.requests[r].tables[1]) == cm.pages_for_tokens(live[r])[1]
        cm.check_invariants()


def test_weights_load_into_fused_layouts(tmp_path):
    W = _write_model(str(tmp_path), F1, seed=3)
    for dtype in (torch.float32, torch.bfloat16):
        model = build_model(config_from_dict(F1).model_spec(), Runtime(dtype, "cpu"))
        assert set(model.weight_specs()) == set(W)
        model.load_from_dir(str(tmp_path))
        f = lambda name: W[name].to(torch.float32)
        att, ssm = model.layers[0].mixer, model.layers[1].mixer
        assert torch.equal(att.w_rows.float(), torch.cat([f("l0.mix.q"), f("l0.mix.k"), f("l0.mix.v")]))
        assert att.bias.dtype == torch.float32 and torch.equal(att.bias, f("l0.mix.pb"))
        assert att.freq.dtype == torch.float32 and tuple(att.freq.shape) == (2, 8)
        want = torch.tensor([10000.0 ** (-2.0 * i / 16) for i in range(8)], dtype=torch.float64)
        assert torch.allclose(att.freq[0].double() + att.freq[1].double(), want, atol=1e-15, rtol=1e-13)
        assert torch.allclose(ssm.neg_a.double(), -torch.exp(W["l1.mix.A_log"].double()), atol=1e-6)
        moe = model.layers[1].feed_forward
        assert tuple(moe.w_gate_up.shape) == (4, 96, 96) and tuple(moe.w_down.shape) == (4, 96, 48)
        for e in range(4):
            assert torch.equal(moe.w_gate_up[e].float(), torch.cat([f("l1.mlp.e%d.gate" % e), f("l1.mlp.e%d.up" % e)]))
            assert torch.equal(moe.w_down[e].float(), f("l1.mlp.e%d.down" % e))
        assert torch.equal(moe.w_router.float(), f("l1.mlp.router"))
        assert torch.equal(moe.shared.w_gate_up.float(), torch.cat([f("l1.mlp.shared.gate"), f("l1.mlp.shared.up")]))
        assert model.layers[2].feed_forward.shared is None
        # the result's norm carries the layer scale; the norm on the input and the token input's norm are plain
        blk = model.layers[0]
        assert torch.allclose(blk.mixer_out_norm.weight.double(), f("l0.norm1b").double() * f("l0.ls1").double(), atol=1e-6)
        assert torch.allclose(blk.feed_forward_out_norm.weight.double(), f("l0.norm2b").double() * f("l0.ls2").double(), atol=1e-6)
        assert torch.equal(blk.mixer_norm.weight, f("l0.norm1")) and torch.equal(blk.side_norm.weight, f("l0.side.norm"))
        assert torch.equal(blk.gates[2][0].float(), f("l0.rg2")) and blk.gates[1][1].dtype == torch.float32
        assert blk.side_table is model.layers[2].side_table or torch.equal(blk.side_table, model.layers[2].side_table)
    missing = {k: v for k, v in W.items() if k != "l0.mix.pb"}
    from safetensors.torch import save_file
    from infinicore_infer_amd.weights.loader import WeightError
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in missing.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        build_model(config_from_dict(F1).model_spec(), Runtime(torch.float32, "cpu")).load_from_dir(str(tmp_path))
    assert "l0.mix.pb" in str(e.value)


def test_what_a_position_sees():
    # window 4, blocks of 3: position 9 sees tokens 6..9; block b is seen once its last token 3b + 2 <= 9 - 4
    assert P.visible(9, 4, 3) == ([6, 7, 8, 9], [0, 1]) and P.visible(8, 4, 3) == ([5, 6, 7, 8], [0])
    assert P.visible(6, 4, 3) == ([3, 4, 5, 6], [0]) and P.visible(5, 4, 3) == ([2, 3, 4, 5], [])
    assert P.visible(12, 4, 3)[1] == [0, 1, 2] and P.visible(11, 4, 3)[1] == [0, 1]
    # tokens 3 and 4 at position 8: out of the window, their block (3..5) not yet wholly before it: not seen at all
    tokens, blocks = P.visible(8, 4, 3)
    assert 4 not in tokens and 1 not in blocks
    assert P.visible(2, 4, 3) == ([0, 1, 2], []) and P.visible(0, 1, 1) == ([0], []) and P.visible(3, 1, 1) == ([3], [0, 1, 2])
    tok, blk = P.seen_masks(3, 4, 3, first=7)             # queries at 7, 8, 9
    assert tok[0].tolist() == [False] * 4 + [True] * 4 + [False] * 2 and blk.tolist() == [[True, False, False], [True, False, False], [True, True, False]]
    tok, blk = P.seen_masks(3, None, 0)
    assert tok.tolist() == [[True, False, False], [True, True, False], [True, True, True]] and blk.shape[1] == 0


def test_the_plain_implementation_is_causal_and_its_parts_do_what_they_say():
    W = P.random_weights(F1, 1)
    toks = list(range(5, 65))
    full = P.forward(F1, W, toks)
    assert torch.allclose(P.forward(F1, W, toks[:17]), full[:17], atol=1e-9)          # what follows changes nothing
    other = P.forward(F1, W, toks[:16] + [99] + toks[17:])
    assert torch.allclose(other[:16], full[:16], atol=1e-9) and not torch.allclose(other[16:], full[16:], atol=1e-3)
    # adjacent pairs turn by position * base^(-2i/dims); entries beyond dims stay
    x = torch.arange(12, dtype=torch.float64).reshape(1, 2, 6) + 1
    y = P.rotate_pairs(x, [5], 4, 100.0)
    a = 5 * 100.0 ** (-2 / 4)
    assert torch.allclose(y[0, 0, 2:4], torch.tensor([3 * math.cos(a) - 4 * math.sin(a), 4 * math.cos(a) + 3 * math.sin(a)], dtype=torch.float64))
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.allclose(y[0, 1, :2], torch.tensor([7 * math.cos(5.0) - 8 * math.sin(5.0), 8 * math.cos(5.0) + 7 * math.sin(5.0)], dtype=torch.float64))
    assert torch.equal(P.rotate_pairs(x, [0], 6, 10.0), x)
    # weights are sigmoids and do not sum to one: with zero scores and no bias every seen item weighs a half
    d, T = 4, 8
    Wa = {"a.q": torch.zeros(d, d, dtype=torch.float64), "a.k": torch.zeros(d, d, dtype=torch.float64), "a.v": torch.eye(d, dtype=torch.float64),
          "a.o": torch.eye(d, dtype=torch.float64), "a.pb": torch.zeros(1, dtype=torch.float64)}
    h = torch.ones(T, d, dtype=torch.float64)
    out = P.pooled_sigmoid_attention(h, Wa, "a.", 1, 1, d, d, 1.0, 3, 2, 0, None)
    seen = [len(P.visible(i, 3, 2)[0]) + len(P.visible(i, 3, 2)[1]) for i in range(T)]
    assert torch.allclose(out[:, 0], torch.tensor([0.5 * n for n in seen], dtype=torch.float64))
    # experts: the weight multiplies the expert's INPUT; the gated unit is not linear, so this differs from weighting the output
    g = torch.Generator().manual_seed(0)
    We = {"m.router": torch.tensor([[4.0, 0.0], [-4.0, 0.0], [0.0, 0.0]], dtype=torch.float64)}
    for e in range(3):
        for n, shape in (("gate", (5, 2)), ("up", (5, 2)), ("down", (2, 5))):
            We["m.e%d.%s" % (e, n)] = torch.randn(*shape, generator=g, dtype=torch.float64)
    hx = torch.tensor([[1.0, 0.3]], dtype=torch.float64)
    s0 = 1 / (1 + math.exp(-4.0))
    want = P.gated_unit(s0 * hx, We, "m.e0.") + P.gated_unit(0.5 * hx, We, "m.e2.")
    assert torch.allclose(P.routed_experts(hx, We, "m.", 3, 2, False), want)
    assert not torch.allclose(want, s0 * P.gated_unit(hx, We, "m.e0.") + 0.5 * P.gated_unit(hx, We, "m.e2."))
    # a tie goes to the lower index
    We["m.router"] = torch.zeros(3, 2, dtype=torch.float64)
    assert torch.allclose(P.routed_experts(hx, We, "m.", 3, 1, False), P.gated_unit(0.5 * hx, We, "m.e0."))
    assert P.run_order({"layers": [0, 1, 2, 3], "loop": {"start": 1, "stop": 3, "times": 3}}) == [
        (0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert torch.allclose(P.gelu_tanh(torch.tensor([1.0], dtype=torch.float64)),
                          torch.tensor([0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715))], dtype=torch.float64))


def test_the_plain_state_space_recurrence_against_its_closed_form():
    g = torch.Generator().manual_seed(0)
    x, w, b = torch.randn(9, 3, generator=g, dtype=torch.float64), torch.randn(3, 4, generator=g, dtype=torch.float64), torch.randn(3, dtype=torch.float64, generator=g)
    pad = torch.cat([torch.zeros(3, 3, dtype=torch.float64), x])
    assert torch.allclose(P.short_conv(x, w, b), b + sum(w[:, k] * pad[k:k + 9] for k in range(4)))


def test_the_scheduler_plans_with_rows_per_block_of_tokens():
    """The scheduler over a cache with a window group and a group of block rows (a stand-in engine on the real cache
    manager): portions, decoding and preemption by recompute give every request its continuation, the block group's pool
    is what runs out first, and every page comes back."""
    from test_scheduler import FakeEngine, _expected, _task
    from infinicore_infer_amd.engine.scheduler import Scheduler

    class TwoGroups(FakeEngine):
        def __init__(self, pages, page_size=4, max_requests=4):
            self.cache = CacheManager([GroupSpec("window", 1, 8, 8, (0,)), GroupSpec("full", 1, 8, None, (0,), stride=2, of_blocks=True)],
                                      pages, page_size, max_requests, None)
            self.history, self.steps = {}, []

        def step(self, entries):
            rows = super().step(entries)
            for e in entries:
                self.cache.trim(e.req_id)
                assert len(self.cache.requests[e.req_id].tables[1]) == self.cache.pages_for_tokens(self.cache.length(e.req_id))[1]
            return rows

    eng = TwoGroups([64, 9])                       # blocks of two tokens, pages of four rows: a page of the block group per 8 tokens
    s = Scheduler(eng, max_batch_tokens=24, chunk_size=16)
    prompts = {i: list(range(i, i + n)) for i, n in enumerate([30, 9, 17])}
    for i, p in prompts.items():
        s.add(_task(i, p, 12))
    while s.has_unfinished():
        s.step()
    done = {t.id: t for t in s.finished}
    for i, p in prompts.items():
        assert done[i].generated == _expected(p, 12)
    assert s.n_preempted > 0                       # 42 + 21 + 29 tokens need 6 + 3 + 4 pages of the block group's nine
    assert eng.cache.free_pages(0) == 64 and eng.cache.free_pages(1) == 9 and not eng.cache.requests
