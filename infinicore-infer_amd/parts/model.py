"""The layered model: an embedding, layers run in the order a list gives, a
final norm and a head.  Built from a ``ModelSpec``; knows no architecture.

Forward of one step (src/models/jiuge/jiuge.cpp:164-168,195-258,261-278 is the
reference's): gather embeddings into the float32 residual stream, run the
schedule, settle the last residual add, then normalise and project only the
rows whose logits are wanted.
"""
from typing import Dict, List

import torch

from ..config.spec import ModelSpec
from ..kernels import ops
from ..weights.loader import WeightSpec, load_weights
from .base import CacheNeed, DeferredRows, Runtime, StreamCopy, build_part


class DecoderModel:
    def __init__(self, spec: ModelSpec, runtime: Runtime):
        self.spec = spec
        self.runtime = runtime
        memo = {}
        self.embedding = build_part("embedding", spec.embedding, runtime, memo)
        self.layers = []
        for ls in spec.layers:
            opt = lambda category, spec: None if spec is None else build_part(category, spec, runtime, memo)
            mixer = opt("mixer", ls.mixer)
            ffn = opt("feed_forward", ls.feed_forward)
            n1 = opt("norm", ls.mixer_norm)
            n2 = opt("norm", ls.feed_forward_norm)
            from .base import _REGISTRY
            try:
                block_cls = _REGISTRY["block"][ls.block.kind]
            except KeyError:
                raise KeyError("no block part of kind %r" % ls.block.kind)
            self.layers.append(block_cls(ls.block.name, runtime, mixer=mixer, mixer_norm=n1, feed_forward=ffn,
                                         feed_forward_norm=n2, **ls.block.params))
        self.final_norm = build_part("norm", spec.final_norm, runtime, memo)
        self.head = build_part("head", spec.head, runtime, memo)
        self.schedule = list(spec.schedule)
        for e in self.schedule:
            if not (0 <= e.layer < len(self.layers)):
                raise ValueError("run order names layer %d, the model has %d" % (e.layer, len(self.layers)))
        writers = {}
        for e in self.schedule:
            if e.writes_cache:
                if e.cache in writers:
                    raise ValueError("cache slot %d is written by two entries of the run order" % e.cache)
                writers[e.cache] = e.layer
        for e in self.schedule:
            if not e.writes_cache and e.cache not in writers:
                raise ValueError("cache slot %d is read but never written" % e.cache)
        self._writers = writers
        self.streams = int(getattr(spec, "residual_streams", 1) or 1)
        if self.streams > 1:
            for l in self.layers:
                if getattr(l, "streams", 1) != self.streams:
                    raise ValueError("block %s keeps %d residual streams, the model %d" % (l.name, getattr(l, "streams", 1), self.streams))
        # an entry that reads another entry's cache must fit what the writer keeps: the same heads and
        # head size, and no more keys than the writer's window holds (pages behind a window are given
        # back and their block-table entries are reused)
        for e in self.schedule:
            if e.writes_cache:
                continue
            wn = self._cache_need_of(writers[e.cache])
            rn = self._cache_need_of(e.layer)
            if not (wn.paged and rn.paged):
                continue
            if (rn.planes, rn.n_kv_heads, rn.head_dim) != (wn.planes, wn.n_kv_heads, wn.head_dim):
                raise ValueError("layer %d reads cache slot %d as %d planes with %d kv heads of %d, its writer (layer %d) "
                                 "keeps %d planes with %d of %d" % (e.layer, e.cache, rn.planes, rn.n_kv_heads, rn.head_dim,
                                                                    writers[e.cache], wn.planes, wn.n_kv_heads, wn.head_dim))
            if wn.window and (not rn.window or rn.window > wn.window):
                raise ValueError("layer %d reads cache slot %d over %s keys, its writer (layer %d) keeps a window of %d"
                                 % (e.layer, e.cache, rn.window or "all", writers[e.cache], wn.window))

    # ---- parts and weights ---------------------------------------------------------
    def all_parts(self):
        seen, out = set(), []

        def walk(p):
            if id(p) in seen:
                return
            seen.add(id(p))
            out.append(p)
            for s in p.sub_parts():
                walk(s)
        walk(self.embedding)
        for l in self.layers:
            walk(l)
        walk(self.final_norm)
        walk(self.head)
        return out

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {}
        for p in self.all_parts():
            for name, s in p.weight_specs().items():
                if name in specs and specs[name] != s:
                    raise ValueError("tensor %s is wanted with two different specs" % name)
                specs[name] = s
        return specs

    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self.all_parts():
            p.load_weights(tensors)

    def load_from_dir(self, model_dir: str) -> None:
        tensors = load_weights(model_dir, self.weight_specs(), self.runtime.dtype, self.runtime.device)
        self.load_weights(tensors)

    # ---- cache needs ------------------------------------------------------------------
    def _cache_need_of(self, layer: int) -> CacheNeed:
        mixer = self.layers[layer].mixer
        return CacheNeed() if mixer is None else mixer.cache_need()       # a layer without a mixer keeps nothing

    def cache_needs(self) -> List[CacheNeed]:
        """One need per cache slot, in slot order."""
        n = self.spec.num_cache_slots()
        needs = [CacheNeed() for _ in range(n)]
        for slot, layer in self._writers.items():
            needs[slot] = self._cache_need_of(layer)
        return needs

    def embedding_cache_need(self) -> CacheNeed:
        """What the embedding keeps per request (the token before a step's first one, for a table of pairs), or nothing."""
        need = getattr(self.embedding, "cache_need", None)
        return need() if need is not None else CacheNeed()

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        for p in self.all_parts():
            for v in vars(p).values():
                if isinstance(v, torch.Tensor) and v.data_ptr() not in seen:
                    seen.add(v.data_ptr())
                    total += v.numel() * v.element_size()
        return total

    # ---- one step ------------------------------------------------------------------------
    def forward(self, ctx):
        """Runs ctx.T tokens; returns float32 logits [len(ctx.want_rows), vocab] or None."""
        T = ctx.T
        shape = (T, self.spec.hidden_size) if self.streams == 1 else (self.streams, T, self.spec.hidden_size)
        x = ctx.ws.buffer("residual", shape, torch.float32)
        if getattr(self.embedding, "takes_context", False):
            pending = self.embedding.forward(ctx.tokens, x, ctx)      # may hand on the stream's copy (StreamCopy)
        else:
            self.embedding.forward(ctx.tokens, x)
            pending = None
        embedded = None
        if any(e.adds_embedding for e in self.schedule):
            # the embedding's output is wanted again later: a pass after the first starts from the stream plus it
            embedded = ctx.ws.buffer("embedded", shape, torch.float32)
            embedded.copy_(x)
        last = len(self.schedule) - 1
        for i, e in enumerate(self.schedule):
            block = self.layers[e.layer]
            if e.adds_embedding:
                if hasattr(pending, "settle"):
                    pending = pending.settle(x, ctx)
                if isinstance(pending, DeferredRows):
                    raise RuntimeError("the embedding's output cannot join a stream whose rows are half normed")
                if pending is not None and not isinstance(pending, StreamCopy):
                    ops.residual_add(x, pending[0], pending[1])
                pending = None
                ops.residual_add(x, embedded, 1.0)
            if hasattr(pending, "settle") and not getattr(block, "accepts_owed_update", False):
                pending = pending.settle(x, ctx)                      # an update only its own kind of block can fuse
            if isinstance(pending, StreamCopy) and not getattr(block, "accepts_stream_copy", False):
                pending = None                                        # nothing is owed; this block makes its own input
            if not block.fuses_successor:
                if isinstance(pending, DeferredRows):
                    raise RuntimeError("block %s was handed half-normed rows it did not ask for" % block.name)
                pending = block.forward(x, pending, ctx, ctx.cache_view(e))
                if ctx.layer_probe is not None:
                    ctx.layer_probe(i, x, pending)
                continue
            # the norm that runs next, if whoever applies it can take its rows half done
            if i < last:
                # (an entry that first adds the embedding's output wants the stream itself, not half-normed rows)
                nxt = self.schedule[i + 1]
                successor = None if nxt.adds_embedding else self.layers[nxt.layer].entry_norm()
            elif ctx.want_rows_identity and getattr(self.head, "accepts_deferred", False):
                successor = self.head.deferred_norm(self.final_norm)
            else:
                successor = None
            pending = block.forward(x, pending, ctx, ctx.cache_view(e), successor=successor)
            if ctx.layer_probe is not None:
                ctx.layer_probe(i, x, pending)
        if hasattr(pending, "settle"):
            pending = pending.settle(x, ctx)
        if ctx.layer_probe is not None:
            ctx.layer_probe(len(self.schedule), x, pending)
        if ctx.n_want == 0:
            return None
        if self.streams > 1:
            # the streams' sum is what the final norm reads
            x = ops.hc_step(x, in_w=self._stream_ones(x), h=ctx.ws.buffer("residual_sum", (T, self.spec.hidden_size), torch.float32))
        if isinstance(pending, DeferredRows):
            return self.head.forward(pending, ctx.want_rows, self.final_norm, ctx)
        if isinstance(pending, StreamCopy):
            pending = None
        if pending is not None:
            ops.residual_add(x, pending[0], pending[1])
        return self.head.forward(x, ctx.want_rows, self.final_norm, ctx)


    def _stream_ones(self, x):
        ones = getattr(self, "_ones", None)
        if ones is None or ones.device != x.device:
            ones = self._ones = torch.ones(self.streams, dtype=torch.float32, device=x.device)
        return ones


def build_model(spec: ModelSpec, runtime: Runtime) -> DecoderModel:
    return DecoderModel(spec, runtime)
