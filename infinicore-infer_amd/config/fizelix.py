"""Typed configuration of the Fizelix decoder, read from config.json.

Keys: ``architecture`` ("Fizelix"), ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``logit_scale``,
``token_side.dim`` (absent: no per-layer token input), ``loop`` {start, stop, times} (layers start..stop-1 run ``times``
times in a row with the same weights, every pass with a cache or state of its own; before every pass but the first the
embedding's output is added to the stream) and ``layers``: a list whose entries give ``type`` ("attention" or "mamba2"),
``mixer`` (the sizes and constants of that mixer) and ``mlp``: null, {kind: "dense", ff} or {kind: "moe", router{experts,
top}, expert{ff}, shared{ff} or absent}.  Tensor names: ``embed``, ``side.embed``, ``final.norm``, ``head`` and per layer i
``l<i>.norm1`` / ``norm1b`` / ``norm2`` / ``norm2b``, ``l<i>.ls1`` / ``ls2``, ``l<i>.rg1`` / ``rg1.b`` / ``rg2`` / ``rg2.b``,
``l<i>.mix.*``, ``l<i>.mlp.*`` (``gate``, ``up``, ``down``; ``router``, ``e<j>.gate`` .., ``shared.gate`` ..),
``l<i>.side.gate`` / ``side.proj`` / ``side.norm``.

The design, layer by layer (x the float32 residual stream, r(z) = z / sqrt(mean(z^2) + eps)):
  x_0 = E[token] * scale
  sublayer q (1 the mixer, 2 the feed-forward):  h = r(x) w_q;  y = f_q(h) * sigmoid(R_q h + b_q);  x <- x + r(y) w_qb ls_q
  after the feed-forward:  g = gelu_tanh(G x) * S[token][i dim : (i + 1) dim];  x <- x + r(P g) w_side
  logits = logit_scale * W_head (r(x) w_final)
The mixers: "attention" rotates adjacent pairs of the first ``rot.dims`` entries of queries and keys, sees the last
``mask.size`` tokens plus the mean key and value of every block of ``mask.pool`` tokens wholly before them, and weighs
what it sees by sigmoid(score + a bias per head) without normalising (``parts/pooled_attention.py``); "mamba2" is the
state-space recurrence (``parts/recurrent.py``).  The routed feed-forward is ``parts/routed_experts.py``.
"""
from dataclasses import dataclass, field
from typing import List, Optional

from .registry import ConfigError, register_architecture
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec

DEFAULT_CONTEXT = 65536        # the design has no limit of its own; a serving cap (max_tokens) replaces this
MIXERS = ("attention", "mamba2")


def _need(d, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json lacks %s%s" % (where, key))
    return d[key]


@dataclass
class FizelixLayer:
    kind: str
    mixer: dict                  # the mixer's sizes and constants as config.json gives them
    mlp: Optional[dict]          # None: the layer has no feed-forward


@dataclass
class FizelixConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: List[FizelixLayer]
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    side_dim: Optional[int] = None                # None: no per-layer token input
    loop: Optional[dict] = None                   # {start, stop, times}
    context_cap: Optional[int] = None
    eos_token_id: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    model_type: str = "Fizelix"

    @classmethod
    def from_dict(cls, cfg: dict, max_tokens: Optional[int] = None) -> "FizelixConfig":
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
            if mlp is not None and not isinstance(mlp, dict):
                raise ConfigError("%smlp must be an object or null" % where)
            layers.append(FizelixLayer(kind, dict(m), dict(mlp) if mlp else None))
        loop = cfg.get("loop")
        if loop:
            loop = {k: int(_need(loop, k, "loop.")) for k in ("start", "stop", "times")}
        side = (cfg.get("token_side") or {}).get("dim")
        eos = cfg.get("eos_token_id", [])
        eos = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        out = cls(vocab_size=int(_need(cfg, "vocab", "")), hidden_size=int(_need(cfg, "width", "")),
                  norm_eps=float(_need(_need(cfg, "norm", ""), "eps", "norm.")), layers=layers,
                  embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                  logit_scale=float(cfg.get("logit_scale", 1.0)), side_dim=int(side) if side else None, loop=loop or None,
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
        if self.side_dim is not None and self.side_dim <= 0:
            raise ConfigError("token_side.dim must be positive")
        n = len(self.layers)
        if self.loop and not (0 <= self.loop["start"] <= self.loop["stop"] <= n and self.loop["times"] >= 1):
            raise ConfigError("loop: 0 <= start <= stop <= %d layers and times >= 1 (got %r)" % (n, self.loop))
        for i, l in enumerate(self.layers):
            self._mixer_spec(i, l)          # names what is missing
            self._ffn_spec(i, l)

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

    def run_order(self):
        """(layer index, does the embedding's output join the stream before it) in the order the layers run: the looped
        stretch ``times`` times in a row, every pass but the first starting from the stream plus the embedding's output."""
        n = len(self.layers)
        if not self.loop:
            return [(i, False) for i in range(n)]
        a, b, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        out = [(i, False) for i in range(a)]
        for rep in range(times):
            out += [(i, rep > 0 and i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

    def to_dict(self) -> dict:
        out = {"architecture": "Fizelix", "vocab": self.vocab_size, "width": self.hidden_size,
               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
               "layers": [{"type": l.kind, "mixer": dict(l.mixer), "mlp": dict(l.mlp) if l.mlp else None} for l in self.layers]}
        if self.side_dim is not None:
            out["token_side"] = {"dim": self.side_dim}
        if self.loop:
            out["loop"] = dict(self.loop)
        return out

    def _mixer_spec(self, i: int, l: FizelixLayer) -> PartSpec:
        d, m, where = self.hidden_size, l.mixer, "layers[%d].mixer." % i
        name = "l%d.mix." % i
        get = lambda k: _need(m, k, where)
        if l.kind == "mamba2":
            return PartSpec("mamba2", name, {
                "hidden_size": d, "heads": int(get("heads")), "head_dim": int(get("vdim")), "state_dim": int(get("state")),
                "groups": int(get("groups")), "conv_taps": int(get("conv")), "norm_groups": int(get("norm_groups")),
                "norm_eps": self.norm_eps})
        mask, rot = m.get("mask") or {}, m.get("rot") or {}
        heads = int(get("heads"))
        size, pool = mask.get("size"), mask.get("pool")
        return PartSpec("pooled_attention", name, {
            "hidden_size": d, "num_heads": heads, "num_kv_heads": int(m.get("kv_heads") or heads), "key_dim": int(get("dim")),
            "value_dim": int(m.get("vdim") or get("dim")), "score_scale": float(get("scale")),
            "window": int(size) if size else None, "block": int(pool) if (pool and size) else None,
            "rot_dims": int(rot.get("dims") or 0), "rot_base": float(rot["base"]) if rot.get("dims") else None,
            "weights": "sigmoid", "head_bias": True})

    def _ffn_spec(self, i: int, l: FizelixLayer) -> Optional[PartSpec]:
        if l.mlp is None:
            return None
        d, where = self.hidden_size, "layers[%d].mlp." % i
        name = "l%d.mlp." % i
        names = {"gate_name": "gate", "up_name": "up", "down_name": "down"}
        kind = l.mlp.get("kind", "dense")
        if kind == "dense":
            ff = int(_need(l.mlp, "ff", where))
            if ff <= 0:
                raise ConfigError("%sff must be positive" % where)
            return PartSpec("swiglu", name, dict(hidden_size=d, intermediate_size=ff, **names))
        if kind != "moe":
            raise ConfigError("%skind %r: this design's feed-forward is dense or moe" % (where, kind))
        router = _need(l.mlp, "router", where)
        experts, top = int(_need(router, "experts", where + "router.")), int(_need(router, "top", where + "router."))
        ff = int(_need(_need(l.mlp, "expert", where), "ff", where + "expert."))
        if not (0 < top <= experts) or ff <= 0:
            raise ConfigError("%s: 0 < top <= experts and a positive expert.ff (got %d, %d, %d)" % (where, top, experts, ff))
        shared = l.mlp.get("shared")
        shared_ff = int(_need(shared, "ff", where + "shared.")) if shared else None
        return PartSpec("routed_experts", name, {
            "hidden_size": d, "experts": experts, "top": top, "expert_size": ff, "shared_size": shared_ff,
            "scores": "sigmoid", "renormalize": False, "weight_on": "input"})

    def model_spec(self) -> ModelSpec:
        d, eps = self.hidden_size, self.norm_eps
        norm = lambda tensor, scale=None: PartSpec("rmsnorm", "", {"size": d, "eps": eps, "tensor": tensor, "scale_tensor": scale})
        layers = []
        for i, l in enumerate(self.layers):
            p = "l%d." % i
            ffn = self._ffn_spec(i, l)
            side = None
            if self.side_dim is not None:
                side = {"table": "side.embed", "table_width": self.side_dim * len(self.layers), "vocab_size": self.vocab_size,
                        "first_column": i * self.side_dim, "dim": self.side_dim,
                        # an RMS norm with a plain weight, whatever the model's norm is
                        "norm": PartSpec("rmsnorm", "", {"size": d, "eps": eps, "tensor": p + "side.norm"})}
            # the norm's weight and the layer scale are one float32 vector for the kernel that adds into the stream
            block = PartSpec("sandwich_gated", p, {
                "hidden_size": d, "mixer_out_norm": norm(p + "norm1b", p + "ls1"),
                "feed_forward_out_norm": None if ffn is None else norm(p + "norm2b", p + "ls2"),
                "gated": True, "side": side})
            layers.append(LayerSpec(block=block, mixer=self._mixer_spec(i, l), mixer_norm=norm(p + "norm1"),
                                    feed_forward=ffn, feed_forward_norm=None if ffn is None else norm(p + "norm2")))
        schedule = [ExecEntry(layer=li, cache=run, writes_cache=True, adds_embedding=again)
                    for run, (li, again) in enumerate(self.run_order())]
        return ModelSpec(
            architecture=self.model_type, vocab_size=self.vocab_size, hidden_size=d, max_positions=self.max_positions,
            embedding=PartSpec("embedding", "embed.", {"vocab_size": self.vocab_size, "hidden_size": d, "tensor": "embed",
                                                       "scale": self.embedding_scale}),
            layers=layers, schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("lm_head", "head.", {"vocab_size": self.vocab_size, "hidden_size": d, "tensor": "head",
                                               "logit_scale": self.logit_scale}),
            eos_token_ids=list(self.eos_token_id), bos_token_id=self.bos_token_id)


register_architecture(["Fizelix", "fizelix"], FizelixConfig)
