"""Host-side parts of the Daborax decoder: its configuration and its errors, layers that run with another layer's
tensors, the model as data, what its parts ask of the cache manager, weights loaded into fused layouts, and the plain
implementation's own properties (causality, the window's two edges, the recurrences against their closed forms)."""
import json
import math

import pytest
import torch

import plain_daborax as P
from test_gpu_daborax import D1, D2, D3, _write_model

from infinicore_infer_amd.config import ConfigError, config_from_dict
from infinicore_infer_amd.parts import Runtime, build_model


def test_config_to_model_spec():
    cfg = config_from_dict(D1)
    spec = cfg.model_spec()
    assert spec.architecture == "Daborax" and spec.vocab_size == 211 and spec.hidden_size == 96 and spec.residual_streams == 1
    # three layers hold tensors; the other three entries of the run order name them and have cache slots of their own
    assert cfg.owners() == [0, 1, 2, 2, 0, 1] and len(spec.layers) == 3
    assert [(e.layer, e.cache, e.writes_cache) for e in spec.schedule] == [(0, 0, True), (1, 1, True), (2, 2, True), (2, 3, True), (0, 4, True), (1, 5, True)]
    assert [l.mixer.kind for l in spec.layers] == ["span_attention", "decay_linear_attention", "mamba2"]
    assert all(l.block.kind == "outnorm_residual" for l in spec.layers)
    a = spec.layers[0].mixer.params
    assert (a["num_heads"], a["num_kv_heads"], a["key_dim"], a["value_dim"], a["window"], a["softcap"]) == (4, 2, 32, 64, 40, 30.0)
    assert (a["sink"], a["qk_norm"], a["qk_norm_weight"], a["qkv_bias"], a["out_bias"], a["softmax_scale"]) == ("learned", "head", False, True, True, 0.18)
    li = spec.layers[1].mixer.params
    assert (li["heads"], li["key_dim"], li["value_dim"], li["decay"]) == (2, 32, 16, [0.9, 0.97])
    n1 = spec.layers[0].mixer_norm.params
    assert (n1["tensor"], n1["scale_tensor"], n1["out_mult"], n1["eps"]) == ("l0.norm1", "l0.ls1", 0.4, 1e-5)
    f = spec.layers[1].feed_forward.params
    assert (f["variant"], f["limit"], f["alpha"], f["intermediate_size"]) == ("clamped", 0.7, 1.702, 64)
    e = spec.embedding.params
    assert (e["scale"], e["sinusoid_base"], e["tensor"]) == (7.0, 10000.0, "embed") and spec.head.params["tensor"] == "head"
    assert "scale_tensor" not in spec.final_norm.params
    assert config_from_dict(cfg.to_dict()).model_spec().layers[0].mixer.params == a
    assert config_from_dict(D1, max_tokens=300).max_positions == 300 and cfg.context_is_open
    # a lender that comes after its borrower; no mask: every earlier key; no cap; a layer without a feed-forward
    late = config_from_dict(D3)
    assert late.owners() == [2, 1, 2, 3, 4] and [e.layer for e in late.model_spec().schedule] == [1, 0, 1, 2, 3]
    assert late.model_spec().layers[0].mixer.params["window"] is None
    plain = config_from_dict(D2).model_spec()
    assert plain.layers[1].mixer.params["softcap"] is None and plain.layers[0].feed_forward is None and plain.layers[0].feed_forward_norm is None
    # a borrower of a borrower runs with the last one's tensors
    chain = json.loads(json.dumps(D1))
    chain["layers"].append(dict(chain["layers"][5], weights_of=5))
    assert config_from_dict(chain).owners() == [0, 1, 2, 2, 0, 1, 1]


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="latent_attention"), "type"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].pop("decay"), "decay"),
    (lambda c: c["layers"][2]["mixer"].pop("norm_groups"), "norm_groups"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "dense"),
    (lambda c: c["layers"][0]["mlp"].pop("limit"), "limit"),
    (lambda c: c.update(layers=[]), "layers"),
    (lambda c: c["layers"][3].update(weights_of=9), "weights_of"),
    (lambda c: c["layers"][3].update(weights_of=0), "type"),
    (lambda c: (c["layers"][0].update(weights_of=4), c["layers"][4].update(weights_of=0)), "circle"),
])
def test_config_errors(change, what):
    cfg = json.loads(json.dumps(D1))
    change(cfg)
    with pytest.raises(ConfigError) as e:
        config_from_dict(cfg)
    assert what in str(e.value)


def test_part_errors():
    from infinicore_infer_amd.parts.base import build_part
    from infinicore_infer_amd.config import PartSpec
    rt = Runtime(torch.float32, "cpu")
    base = {"hidden_size": 16, "heads": 2, "key_dim": 8, "value_dim": 8, "decay": [0.5, 0.5], "norm_eps": 1e-5}
    for bad in ({"decay": [0.5]}, {"decay": [0.5, 1.5]}, {"value_dim": 300}, {"key_dim": 600}):
        with pytest.raises(ValueError):
            build_part("mixer", PartSpec("decay_linear_attention", "m.", dict(base, **bad)), rt)
    with pytest.raises(ValueError):
        build_part("feed_forward", PartSpec("swiglu", "f.", {"hidden_size": 8, "intermediate_size": 8, "variant": "clamped"}), rt)
    att = {"hidden_size": 16, "num_heads": 2, "num_kv_heads": 1, "key_dim": 8, "value_dim": 8, "softmax_scale": 0.3}
    for bad in ({"sink": "loud"}, {"softcap": -1.0}, {"qk_norm": "row", "qk_norm_weight": False}):
        with pytest.raises(ValueError):
            build_part("mixer", PartSpec("span_attention", "a.", dict(att, **bad)), rt)


def test_cache_needs_of_the_mixers():
    model = build_model(config_from_dict(D1).model_spec(), Runtime(torch.float32, "cpu"))
    needs = model.cache_needs()
    assert [n.kind for n in needs] == ["kv", "state", "state", "state", "kv", "state"]
    att, lin, ssm = needs[0], needs[1], needs[2]
    assert (att.planes, att.n_kv_heads, att.plane_dims, att.window, att.keep_first) == (2, 2, (32, 64), 40, 0)
    assert lin.state_shape == (2 * 32 * 16,) and lin.state_dtype == torch.float32
    assert ssm.state_shape == (4 * 24 * 16 + 3 * (64 + 2 * 2 * 24),) and needs[3] == ssm and needs[4] == att and needs[5] == lin


def test_weights_load_into_fused_layouts(tmp_path):
    W = _write_model(str(tmp_path), D1, seed=3)
    for dtype in (torch.float32, torch.bfloat16):
        model = build_model(config_from_dict(D1).model_spec(), Runtime(dtype, "cpu"))
        assert set(model.weight_specs()) == set(W)
        model.load_from_dir(str(tmp_path))
        att, lin, ssm = (model.layers[i].mixer for i in (0, 1, 2))
        f = lambda name: W[name].to(torch.float32)
        assert torch.equal(att.w_rows.float(), torch.cat([f("l0.mix.q"), f("l0.mix.k"), f("l0.mix.v")]))
        assert torch.equal(att.b_rows, torch.cat([f("l0.mix.q.b"), f("l0.mix.k.b"), f("l0.mix.v.b")]))
        assert att.sinks.dtype == torch.float32 and torch.equal(att.sinks, f("l0.mix.sink")) and att.q_norm is None
        assert torch.equal(lin.w_rows.float(), torch.cat([f("l1.mix.v"), f("l1.mix.k"), f("l1.mix.q"), f("l1.mix.g")]))
        assert lin.decay.dtype == torch.float32 and lin.decay.tolist() == [torch.tensor(a).float().item() for a in (0.9, 0.97)]
        assert torch.allclose(ssm.neg_a.double(), -torch.exp(W["l2.mix.A_log"].double()), atol=1e-6)
        # the norm's weight, the layer scale and the residual multiplier are one float32 vector
        n1 = model.layers[0].mixer_norm
        assert n1.weight.dtype == torch.float32 and torch.allclose(n1.weight.double(), f("l0.norm1").double() * f("l0.ls1").double() * 0.4, atol=1e-6)
        assert torch.equal(model.final_norm.weight, f("final.norm"))
        ff = model.layers[0].feed_forward
        assert torch.equal(ff.w_gate_up.float(), torch.cat([f("l0.mlp.gate"), f("l0.mlp.up")]))
    missing = {k: v for k, v in W.items() if k != "l0.mix.sink"}
    from safetensors.torch import save_file
    from infinicore_infer_amd.weights.loader import WeightError
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in missing.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        build_model(config_from_dict(D1).model_spec(), Runtime(torch.float32, "cpu")).load_from_dir(str(tmp_path))
    assert "l0.mix.sink" in str(e.value)


def test_the_plain_implementation_is_causal_and_its_window_has_two_edges():
    W = P.random_weights(D1, 1)
    toks = list(range(5, 65))
    full = P.forward(D1, W, toks)
    assert torch.allclose(P.forward(D1, W, toks[:17]), full[:17], atol=1e-9)          # what follows changes nothing
    other = P.forward(D1, W, toks[:16] + [99] + toks[17:])
    assert torch.allclose(other[:16], full[:16], atol=1e-9) and not torch.allclose(other[16:], full[16:], atol=1e-3)
    m = P.seen(3, 10, 4, first=7)                 # queries at positions 7, 8, 9 with a window of 4
    assert m[0].tolist() == [False] * 4 + [True] * 4 + [False] * 2 and m[2].tolist() == [False] * 6 + [True] * 4
    assert P.seen(2, 3, None).tolist() == [[True, False, False], [True, True, False]]
    # the sink takes its share and has no value: the weights sum to less than one; a far larger sink takes nearly all
    s = torch.zeros(1, 4, dtype=torch.float64)
    w = P.sink_softmax(s, torch.ones(1, 4, dtype=torch.bool), 0.0)
    assert torch.allclose(w, torch.full((1, 4), 0.2, dtype=torch.float64))
    assert float(P.sink_softmax(s, torch.ones(1, 4, dtype=torch.bool), 20.0).sum()) < 1e-7
    # the cap bounds the score, not the sink
    big = torch.tensor([[1000.0, 0.0]], dtype=torch.float64)
    w = P.sink_softmax(big, torch.ones(1, 2, dtype=torch.bool), 5.0, softcap=5.0)
    assert torch.allclose(w[0, 0], torch.tensor(math.exp(5 * math.tanh(200.0)) / (math.exp(5.0) + math.exp(5 * math.tanh(200.0)) + 1.0), dtype=torch.float64))


def test_the_plain_recurrences_against_their_closed_forms():
    g = torch.Generator().manual_seed(0)
    x, w, b = torch.randn(9, 3, generator=g, dtype=torch.float64), torch.randn(3, 4, generator=g, dtype=torch.float64), torch.randn(3, dtype=torch.float64, generator=g)
    pad = torch.cat([torch.zeros(3, 3, dtype=torch.float64), x])
    assert torch.allclose(P.short_conv(x, w, b), b + sum(w[:, k] * pad[k:k + 9] for k in range(4)))
    # linear attention is a decayed sum over earlier tokens: o_t = sum_j decay^(t-j) (q_t . k_j) v_j
    T, d, heads, dk, dv = 7, 6, 2, 3, 4
    W = {"m.q": torch.randn(heads * dk, d, generator=g, dtype=torch.float64), "m.k": torch.randn(heads * dk, d, generator=g, dtype=torch.float64),
         "m.v": torch.randn(heads * dv, d, generator=g, dtype=torch.float64), "m.g": torch.zeros(heads * dv, d, dtype=torch.float64),
         "m.norm": torch.ones(heads * dv, dtype=torch.float64), "m.o": torch.eye(heads * dv, dtype=torch.float64)}
    h = torch.randn(T, d, generator=g, dtype=torch.float64)
    decay = [0.5, 1.0]
    q, k, v = (P.silu(h @ W["m." + n].T) for n in "qkv")
    o = torch.zeros(T, heads, dv, dtype=torch.float64)
    for hd in range(heads):
        for t in range(T):
            for j in range(t + 1):
                o[t, hd] += decay[hd] ** (t - j) * (q[t, hd * dk:(hd + 1) * dk] @ k[j, hd * dk:(hd + 1) * dk]) * v[j, hd * dv:(hd + 1) * dv]
    want = P.unit_rms(o.reshape(T, -1), 1e-6) * 0.5                      # gate zero: sigmoid is a half
    assert torch.allclose(P.lightning_mixer(h, W, "m.", heads, dk, dv, decay, 1e-6), want)
    # the gated unit: inside the limits it is g sigmoid(1.702 g) (u + 1); beyond them the limits stand in
    Wf = {"f.gate": torch.eye(2, dtype=torch.float64), "f.up": torch.eye(2, dtype=torch.float64), "f.down": torch.eye(2, dtype=torch.float64)}
    y = P.clamped_glu(torch.tensor([[0.5, 9.0], [-9.0, -9.0]], dtype=torch.float64), Wf, "f.", 2.0)
    sg = lambda z: 1 / (1 + math.exp(-1.702 * z))
    assert torch.allclose(y, torch.tensor([[0.5 * sg(0.5) * 1.5, 2.0 * sg(2.0) * 3.0], [-9.0 * sg(-9.0) * -1.0, -9.0 * sg(-9.0) * -1.0]], dtype=torch.float64))
    pv = P.position_vectors(3, 6, torch.float64, first=4)
    assert torch.allclose(pv[1, 2], torch.tensor(math.sin(5 * 10000 ** (-2 / 6)), dtype=torch.float64)) and torch.allclose(pv[1, 3], torch.tensor(math.cos(5 * 10000 ** (-2 / 6)), dtype=torch.float64))
