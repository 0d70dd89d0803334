"""Typed configuration of the Daborax decoder, read from config.json.

Keys: ``architecture`` ("Daborax"), ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``residual_mult`` and
``layers``: a list whose entries give ``type`` ("attention", "lightning" or "mamba2"), ``mixer`` (the sizes and constants
of that mixer), ``mlp`` ({kind: "dense", ff, limit} or null) and optionally ``weights_of``: j, which says that the layer
has no tensors of its own and runs with layer j's (mixer, feed-forward, norms and layer scales) on a cache or state of
its own.  Tensor names: ``embed``, ``final.norm``, ``head`` and per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.ls1``,
``l<i>.ls2``, ``l<i>.mix.*``, ``l<i>.mlp.gate`` / ``.up`` / ``.down``.

The design, layer by layer (x the float32 residual stream, r(z) = z / sqrt(mean(z^2) + eps), m = residual_mult):
  x_0 = E[token] * scale + s(p),  s(p)[2i] = sin(p 10000^(-2i/width)),  s(p)[2i+1] = cos(p 10000^(-2i/width))
  x <- x + m * r(mixer(x)) * w_norm1 * ls1;   x <- x + m * r(ffn(x)) * w_norm2 * ls2      (second half if mlp)
  ffn(h) = W_down (g sigmoid(1.702 g) (u + 1)),  g = min(W_gate h, limit),  u = clamp(W_up h, -limit, limit)
  logits = W_head (r(x) w_final)
The mixers: "attention" is softmax attention without rotation over a window of ``mask.size`` keys, with biases on q, k, v
and the output, queries and keys brought to unit root mean square per head (no weight), the score capped by
``softcap * tanh(score / softcap)`` and a learned sink per head in the softmax's denominator
(``parts/span_attention.py``); "lightning" is linear attention with a fixed decay per head and "mamba2" a state-space
recurrence (``parts/recurrent.py``).
"""
from dataclasses import dataclass, field
from typing import List, Optional

from .registry import ConfigError, register_architecture
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec

SINUSOID_BASE = 10000.0
GLU_SIGMOID_SLOPE = 1.702      # g * sigmoid(1.702 g): fixed by the design
DEFAULT_CONTEXT = 65536        # the design has no limit of its own; a serving cap (max_tokens) replaces this
MIXERS = ("attention", "lightning", "mamba2")


def _need(d, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json lacks %s%s" % (where, key))
    return d[key]


@dataclass
class DaboraxLayer:
    kind: str
    mixer: dict                  # the mixer's sizes and constants as config.json gives them
    ff: Optional[int]            # None: the layer has no feed-forward
    ff_limit: Optional[float]
    weights_of: Optional[int]    # the layer whose tensors this one runs with; None: its own


@dataclass
class DaboraxConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    layers: List[DaboraxLayer]
    context_cap: Optional[int] = None
    eos_token_id: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    model_type: str = "Daborax"

    @classmethod
    def from_dict(cls, cfg: dict, max_tokens: Optional[int] = None) -> "DaboraxConfig":
        raw_layers = _need(cfg, "layers", "")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, l in enumerate(raw_layers):
            where = "layers[%d]." % i
            kind = _need(l, "type", where)
            if kind not in MIXERS:
                raise ConfigError("%stype %r: this design has the mixers %s" % (where, kind, ", ".join(MIXERS)))
            m = _need(l, "mixer", where)
            if not isinstance(m, dict):
                raise ConfigError("%smixer must be an object" % where)
            mlp = l.get("mlp")
            ff = limit = None
            if mlp:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError("%smlp.kind %r: this design's feed-forward is dense" % (where, mlp.get("kind")))
                ff = int(_need(mlp, "ff", where + "mlp."))
                limit = float(_need(mlp, "limit", where + "mlp."))
            src = l.get("weights_of")
            layers.append(DaboraxLayer(kind, dict(m), ff, limit, None if src is None else int(src)))
        eos = cfg.get("eos_token_id", [])
        eos = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        out = cls(vocab_size=int(_need(cfg, "vocab", "")), hidden_size=int(_need(cfg, "width", "")),
                  norm_eps=float(_need(_need(cfg, "norm", ""), "eps", "norm.")),
                  embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                  residual_mult=float(cfg.get("residual_mult", 1.0)), layers=layers,
                  context_cap=int(max_tokens) if max_tokens is not None else None,
                  eos_token_id=[int(e) for e in eos], bos_token_id=cfg.get("bos_token_id"))
        out.validate()
        return out

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.context_cap is not None and self.context_cap <= 0:
            raise ConfigError("max_tokens (the cap on the context) must be positive")
        for i, l in enumerate(self.layers):
            if l.ff is not None and (l.ff <= 0 or not l.ff_limit > 0):
                raise ConfigError("layers[%d]: mlp.ff and mlp.limit must be positive" % i)
            if l.weights_of is not None:
                j = l.weights_of
                if not 0 <= j < len(self.layers) or j == i:
                    raise ConfigError("layers[%d]: weights_of names layer %r; the model has layers 0..%d" % (i, j, len(self.layers) - 1))
            else:
                self._mixer_spec(i, l)          # names what is missing
        for i, o in enumerate(self.owners()):
            if self.layers[o].kind != self.layers[i].kind:
                raise ConfigError("layers[%d] is of type %r and cannot run with the tensors of layer %d (%r)"
                                  % (i, self.layers[i].kind, o, self.layers[o].kind))

    @property
    def max_positions(self) -> int:
        return self.context_cap if self.context_cap is not None else DEFAULT_CONTEXT

    context_is_open = True      # positions are bounded by the serving cap or the cache pool only

    @property
    def default_dtype(self) -> str:
        return "bfloat16"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def owners(self) -> List[int]:
        """For every layer of the configuration, the layer whose tensors it runs with (itself, mostly).  A layer that
        names one which names another runs with the last one's; its sizes and constants are that layer's."""
        out = []
        for i, l in enumerate(self.layers):
            seen = {i}
            while l.weights_of is not None:
                i = l.weights_of
                if i in seen:
                    raise ConfigError("layers: weights_of runs in a circle through layer %d" % i)
                seen.add(i)
                l = self.layers[i]
            out.append(i)
        return out

    def to_dict(self) -> dict:
        layers = []
        for l in self.layers:
            e = {"type": l.kind, "mixer": dict(l.mixer),
                 "mlp": {"kind": "dense", "ff": l.ff, "limit": l.ff_limit} if l.ff is not None else None}
            if l.weights_of is not None:
                e["weights_of"] = l.weights_of
            layers.append(e)
        return {"architecture": "Daborax", "vocab": self.vocab_size, "width": self.hidden_size,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                "residual_mult": self.residual_mult, "layers": layers}

    def _mixer_spec(self, i: int, l: DaboraxLayer) -> PartSpec:
        d, m, where = self.hidden_size, l.mixer, "layers[%d].mixer." % i
        name = "l%d.mix." % i
        get = lambda k: _need(m, k, where)
        if l.kind == "mamba2":
            return PartSpec("mamba2", name, {
                "hidden_size": d, "heads": int(get("heads")), "head_dim": int(get("vdim")), "state_dim": int(get("state")),
                "groups": int(get("groups")), "conv_taps": int(get("conv")), "norm_groups": int(get("norm_groups")),
                "norm_eps": self.norm_eps})
        if l.kind == "lightning":
            decay = get("decay")
            if not isinstance(decay, list):
                raise ConfigError("%sdecay must be a list with one number per head" % where)
            return PartSpec("decay_linear_attention", name, {
                "hidden_size": d, "heads": int(get("heads")), "key_dim": int(get("dim")),
                "value_dim": int(m.get("vdim") or get("dim")), "decay": [float(a) for a in decay], "norm_eps": self.norm_eps})
        mask = m.get("mask") or {}
        size = mask.get("size")
        heads = int(get("heads"))
        return PartSpec("span_attention", name, {
            "hidden_size": d, "num_heads": heads, "num_kv_heads": int(m.get("kv_heads") or heads), "key_dim": int(get("dim")),
            "value_dim": int(m.get("vdim") or get("dim")), "softmax_scale": float(get("scale")),
            "window": int(size) if size else None, "sink": "learned", "softcap": float(m["softcap"]) if m.get("softcap") else None,
            "qk_norm": "head", "qk_norm_weight": False, "qk_norm_eps": self.norm_eps, "qkv_bias": True, "out_bias": True})

    def model_spec(self) -> ModelSpec:
        d, eps = self.hidden_size, self.norm_eps
        # norm weight, layer scale and the residual multiplier are one float32 vector for the kernel that adds into the stream
        into_stream = lambda tensor, scale: PartSpec("rmsnorm", "", {"size": d, "eps": eps, "tensor": tensor, "scale_tensor": scale,
                                                                    "out_mult": self.residual_mult})
        layers, index = [], {}
        for i, l in enumerate(self.layers):
            if l.weights_of is not None:
                continue
            p = "l%d." % i
            index[i] = len(layers)
            layers.append(LayerSpec(
                block=PartSpec("outnorm_residual", p, {}), mixer=self._mixer_spec(i, l),
                mixer_norm=into_stream(p + "norm1", p + "ls1"),
                feed_forward=None if l.ff is None else PartSpec("swiglu", p + "mlp.", {
                    "hidden_size": d, "intermediate_size": l.ff, "gate_name": "gate", "up_name": "up", "down_name": "down",
                    "variant": "clamped", "limit": l.ff_limit, "alpha": GLU_SIGMOID_SLOPE}),
                feed_forward_norm=None if l.ff is None else into_stream(p + "norm2", p + "ls2")))
        # every layer of the configuration is one entry of the run order with a cache slot of its own; a layer that
        # runs with another's tensors names that layer
        schedule = [ExecEntry(layer=index[o], cache=run, writes_cache=True) for run, o in enumerate(self.owners())]
        return ModelSpec(
            architecture=self.model_type, vocab_size=self.vocab_size, hidden_size=d, max_positions=self.max_positions,
            embedding=PartSpec("embedding", "embed.", {"vocab_size": self.vocab_size, "hidden_size": d, "tensor": "embed",
                                                       "scale": self.embedding_scale, "sinusoid_base": SINUSOID_BASE}),
            layers=layers, schedule=schedule,
            final_norm=PartSpec("rmsnorm", "", {"size": d, "eps": eps, "tensor": "final.norm"}),
            head=PartSpec("lm_head", "head.", {"vocab_size": self.vocab_size, "hidden_size": d, "tensor": "head"}),
            eos_token_ids=list(self.eos_token_id), bos_token_id=self.bos_token_id)


register_architecture(["Daborax", "daborax"], DaboraxConfig)
