"""Pre-norm residual block: x += a * mixer(norm1(x)); x += a * ffn(norm2(x))
(the second half only when the layer has a feed-forward: a stack of mixers alone leaves it out),
with a = scale_depth / sqrt(num_layers) (scripts/jiuge.py:109-114; the
reference folds it into o_proj and down_proj, jiuge.py:284-299,335-350, here it
is a float32 factor of the residual add).  The layer body is
src/models/jiuge/jiuge.cpp:195-258.

The residual stream is float32.  Each add is fused with the norm that follows
it: the block leaves its last add pending for whoever normalises next.  For
few rows the add and the norm go further, into the products on either side
(``ResidualTail`` / ``DeferredRows``): then a layer is six kernels, not eight.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Block, DeferredRows, ResidualTail, StreamCopy, register_part


@register_part("block", "prenorm_residual")
class PreNormResidualBlock(Block):
    graph_safe = True
    fuses_successor = True

    def __init__(self, name, runtime, mixer=None, mixer_norm=None, feed_forward=None, feed_forward_norm=None,
                 residual_scale: float = 1.0):
        super().__init__(name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm)
        if mixer is None or mixer_norm is None:
            raise ValueError("block %s: a pre-norm residual block needs a mixer and its norm" % name)
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("block %s: a feed-forward and its norm come together, or neither" % name)
        self.residual_scale = float(residual_scale)

    def entry_norm(self):
        """The norm applied to the incoming stream, if the mixer can take its rows half done."""
        return self.mixer_norm if getattr(self.mixer, "accepts_deferred", False) else None

    def _tail(self, producer, consumer_ok, norm, x):
        """The request to fuse (add, norm) into the producer's last projection, when all three agree."""
        if not (getattr(producer, "fuses_tail", False) and consumer_ok and norm is not None):
            return None
        d = norm.deferred()
        return None if d is None else ResidualTail(x, self.residual_scale, d[0], d[1])

    def native_desc(self):
        """The layer for the native step function, when it is this arrangement of parts that all have
        a native description themselves (attention, SwiGLU, RMS norms)."""
        from ..kernels.lib import IcAttention, IcLayer, IcNorm, IcSwiGLU
        if not self._forward_is(PreNormResidualBlock) or self.feed_forward is None:
            return None
        descs = [p.native_desc() for p in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)]
        if not (isinstance(descs[0], IcNorm) and isinstance(descs[1], IcAttention) and isinstance(descs[2], IcNorm)
                and isinstance(descs[3], IcSwiGLU)):
            return None
        return IcLayer(descs[0], descs[1], descs[2], descs[3], self.residual_scale)

    def forward(self, x, pending, ctx, cache, successor=None):
        if isinstance(pending, DeferredRows):
            h = pending                               # the add is done; the mixer applies the row factors
        else:
            h = ctx.ws.buffer("normed", tuple(x.shape), self.runtime.dtype)
            if pending is None:
                self.mixer_norm.forward(x, h)
            else:
                self.mixer_norm.forward_add(x, pending[0], pending[1], h)
        if self.feed_forward is None:                 # a layer of a mixer alone: its add is what the layer leaves owed
            tail = self._tail(self.mixer, True, successor, x)
            y = self.mixer.forward(h, ctx, cache, tail=tail) if tail is not None else self.mixer.forward(h, ctx, cache)
            return y if isinstance(y, DeferredRows) else (y, self.residual_scale)
        tail = self._tail(self.mixer, getattr(self.feed_forward, "accepts_deferred", False), self.feed_forward_norm, x)
        y = self.mixer.forward(h, ctx, cache, tail=tail) if tail is not None else self.mixer.forward(h, ctx, cache)
        if isinstance(y, DeferredRows):
            h = y
        else:
            h = ctx.ws.buffer("normed", tuple(x.shape), self.runtime.dtype)
            self.feed_forward_norm.forward_add(x, y, self.residual_scale, h)
        tail = self._tail(self.feed_forward, True, successor, x)
        y = self.feed_forward.forward(h, ctx, tail=tail) if tail is not None else self.feed_forward.forward(h, ctx)
        if isinstance(y, DeferredRows):
            return y
        return (y, self.residual_scale)


@register_part("block", "outnorm_residual")
class OutputNormResidualBlock(Block):
    """x += norm1(mixer(x)); x += norm2(ffn(x)): the sublayers read the residual stream itself and the norm sits on
    their OUTPUT, on the way back into the stream (the second half only when the layer has a feed-forward).

    The stream is float32; a sublayer's products want it in the compute dtype, so the kernel that updates the stream
    (``forward_into_stream`` of the norm part) writes that copy along and the block hands it to the next one as
    ``StreamCopy``: a layer is its products, the attention kernels and two row kernels.  A mixer that keeps its last
    projection's bias back (``defers_bias``) has it added inside the norm kernel, before the sum of squares."""
    graph_safe = True
    accepts_stream_copy = True

    def __init__(self, name, runtime, mixer=None, mixer_norm=None, feed_forward=None, feed_forward_norm=None):
        super().__init__(name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm)
        if mixer is None or mixer_norm is None:
            raise ValueError("block %s: an output-norm residual block needs a mixer and its norm" % name)
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("block %s: a feed-forward and its norm come together, or neither" % name)
        for n in (mixer_norm, feed_forward_norm):
            if n is not None and not hasattr(n, "forward_into_stream"):
                raise ValueError("block %s: norm part %s cannot normalise a sublayer's output into the stream"
                                 % (name, type(n).__name__))

    def _copy_buffer(self, x, ctx):
        return None if self.runtime.dtype == x.dtype else ctx.ws.buffer("stream_copy", tuple(x.shape), self.runtime.dtype)

    def forward(self, x, pending, ctx, cache):
        if isinstance(pending, StreamCopy):
            h = pending.values
        else:
            if pending is not None:
                from ..kernels import ops
                ops.residual_add(x, pending[0], pending[1])
            h = self._copy_buffer(x, ctx)
            h = x if h is None else h.copy_(x)
        if getattr(self.mixer, "defers_bias", False):
            y = self.mixer.forward(h, ctx, cache, defer_bias=True)
            bias = self.mixer.deferred_bias()
        else:
            y, bias = self.mixer.forward(h, ctx, cache), None
        copy = self._copy_buffer(x, ctx)
        self.mixer_norm.forward_into_stream(y, x, copy=copy, bias=bias)
        h = x if copy is None else copy
        if self.feed_forward is not None:
            y = self.feed_forward.forward(h, ctx)
            self.feed_forward_norm.forward_into_stream(y, x, copy=copy)
        return StreamCopy(h)


class OwedStreamWrite:
    """The write of a sublayer's result into several residual streams, still owed: the next read of the streams (the
    next sublayer's input, in whichever block) does it in the same kernel.  Whoever cannot, settles it."""

    def __init__(self, y, mix, out_w):
        self.y, self.mix, self.out_w = y, mix, out_w

    def settle(self, x, ctx=None):
        ops.hc_step(x if x.dim() == 3 else x.unsqueeze(0), y=self.y, mix=self.mix, out_w=self.out_w)
        return None


@register_part("block", "hyper_connections")
class HyperConnectionBlock(Block):
    """Pre-norm sublayers over ``streams`` float32 copies of the residual stream x_1..x_S ([S, T, d]).  Sublayer q
    (1: the mixer, 2: the feed-forward) reads u = sum_s in_q[s] x_s, computes y = f(norm_q(u)), and rewrites all streams
    at once from the old ones: x_t <- sum_s mix_q[s, t] x_s + out_q[t] y.  Tensors: ``hc<q>.in`` [S], ``hc<q>.out`` [S],
    ``hc<q>.mix`` [S, S] ([from, to]), held in float32.  One row kernel per sublayer does the write owed by the
    sublayer before, the read, and the norm."""
    graph_safe = True
    accepts_owed_update = True

    def __init__(self, name, runtime, mixer=None, mixer_norm=None, feed_forward=None, feed_forward_norm=None, streams: int = 2):
        super().__init__(name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm)
        if mixer is None or mixer_norm is None:
            raise ValueError("block %s: a hyper-connection block needs a mixer and its norm" % name)
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("block %s: a feed-forward and its norm come together, or neither" % name)
        for n in (mixer_norm, feed_forward_norm):
            if n is not None and n.deferred() is None:
                raise ValueError("block %s: norm part %s is not a weighted RMS norm" % (name, type(n).__name__))
        self.streams = int(streams)
        if not 1 <= self.streams <= 8:
            raise ValueError("block %s: 1..8 residual streams (got %d)" % (name, self.streams))
        self.hc = {}

    def _subs(self):
        return (1, 2) if self.feed_forward is not None else (1,)

    def weight_specs(self):
        S, specs = self.streams, {}
        for q in self._subs():
            p = "%shc%d." % (self.name, q)
            # (random-weights mode draws them around means that keep the streams' size: the read and the mix average)
            specs[p + "in"] = WeightSpec((S,), "vector", mean=1.0 / S)
            specs[p + "out"] = WeightSpec((S,), "vector")
            specs[p + "mix"] = WeightSpec((S, S), "vector", mean=1.0 / S)
        return specs

    def load_weights(self, tensors):
        for q in self._subs():
            p = "%shc%d." % (self.name, q)
            self.hc[q] = tuple(tensors[p + k].to(torch.float32).contiguous() for k in ("in", "out", "mix"))

    def _read(self, x, pending, q, norm, ctx):
        """The sublayer's input: the owed write (if any), the read and the norm in one kernel."""
        T, d = x.shape[1], x.shape[2]
        h = ctx.ws.buffer("normed", (T, d), self.runtime.dtype)
        w, eps = norm.deferred()
        if isinstance(pending, OwedStreamWrite):
            ops.hc_step(x, y=pending.y, mix=pending.mix, out_w=pending.out_w, in_w=self.hc[q][0], norm_w=w, eps=eps, h=h)
        else:
            ops.hc_step(x, in_w=self.hc[q][0], norm_w=w, eps=eps, h=h)
        return h

    def forward(self, x, pending, ctx, cache):
        if x.dim() == 2 and self.streams == 1:
            x = x.unsqueeze(0)                        # one stream: the model keeps it as [T, d]
        if x.dim() != 3 or x.shape[0] != self.streams:
            raise RuntimeError("block %s wants the residual stream as [%d, T, d]" % (self.name, self.streams))
        if pending is not None and not isinstance(pending, OwedStreamWrite):
            if isinstance(pending, StreamCopy):
                pending = None
            else:
                raise RuntimeError("block %s was handed a pending add of another kind of block" % self.name)
        h = self._read(x, pending, 1, self.mixer_norm, ctx)
        y = self.mixer.forward(h, ctx, cache)
        pending = OwedStreamWrite(y, self.hc[1][2], self.hc[1][1])
        if self.feed_forward is not None:
            h = self._read(x, pending, 2, self.feed_forward_norm, ctx)
            y = self.feed_forward.forward(h, ctx)
            pending = OwedStreamWrite(y, self.hc[2][2], self.hc[2][1])
        return pending


@register_part("block", "sandwich_gated")
class SandwichGatedBlock(Block):
    """Norms on both sides of every sublayer, a gate on its result, and an optional per-layer token input:

        h = norm_in(x);  y = f(h) * sigmoid(R h + b);  x += norm_out(y)            (f the mixer, then the feed-forward)
        g = gelu_tanh(G x) * S[token][c0 : c0 + dim];  x += side_norm(P g)          (after the last sublayer)

    ``mixer_out_norm`` / ``feed_forward_out_norm``: the specs of the norms on the results (a layer scale rides in their
    weight).  ``gated``: the tensors ``rg1`` [d, d], ``rg1.b`` [d] (``rg2``.. for the feed-forward); the gate is made from
    the sublayer's input h and applied before the result's norm.  ``side``: None or {table, table_width, vocab_size,
    first_column, dim, norm}: the tensors ``side.gate`` [dim, d], ``side.proj`` [d, dim] and a table shared by the layers,
    of which this layer reads ``dim`` columns from ``first_column``; the gate is made from the stream itself.

    The gate, the result's norm, the layer scale and the add into the float32 stream are one row kernel
    (``ops.gated_norm_into_stream``), which also writes the stream's copy in the compute dtype when the token input wants it."""
    graph_safe = True

    def __init__(self, name, runtime, mixer=None, mixer_norm=None, feed_forward=None, feed_forward_norm=None,
                 hidden_size: int = 0, mixer_out_norm=None, feed_forward_out_norm=None, gated: bool = True, side=None):
        super().__init__(name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm)
        from .base import build_part
        if mixer is None or mixer_norm is None or mixer_out_norm is None:
            raise ValueError("block %s: a sandwich block needs a mixer and the norms before and after it" % name)
        if not ((feed_forward is None) == (feed_forward_norm is None) == (feed_forward_out_norm is None)):
            raise ValueError("block %s: a feed-forward and its two norms come together, or none of them" % name)
        self.hidden_size = int(hidden_size)
        if self.hidden_size <= 0:
            raise ValueError("block %s: hidden_size must be positive" % name)
        self.mixer_out_norm = build_part("norm", mixer_out_norm, runtime)
        self.feed_forward_out_norm = None if feed_forward_out_norm is None else build_part("norm", feed_forward_out_norm, runtime)
        for n in (self.mixer_out_norm, self.feed_forward_out_norm):
            if n is not None and n.deferred() is None:
                raise ValueError("block %s: norm part %s is not a weighted RMS norm" % (name, type(n).__name__))
        self.gated = bool(gated)
        self.side = dict(side) if side else None
        self.side_norm = build_part("norm", self.side["norm"], runtime) if self.side else None
        if self.side_norm is not None and self.side_norm.deferred() is None:
            raise ValueError("block %s: norm part %s is not a weighted RMS norm" % (name, type(self.side_norm).__name__))
        self.gates = {}
        self.side_gate = self.side_proj = self.side_table = None

    def sub_parts(self):
        extra = (self.mixer_out_norm, self.feed_forward_out_norm, self.side_norm)
        return super().sub_parts() + tuple(p for p in extra if p is not None)

    def _subs(self):
        return (1, 2) if self.feed_forward is not None else (1,)

    def weight_specs(self):
        d, specs = self.hidden_size, {}
        if self.gated:
            for q in self._subs():
                specs["%srg%d" % (self.name, q)] = WeightSpec((d, d))
                specs["%srg%d.b" % (self.name, q)] = WeightSpec((d,), "vector", mean=0.0)
        if self.side:
            s = self.side
            specs[s["table"]] = WeightSpec((s["vocab_size"], s["table_width"]))
            specs[self.name + "side.gate"] = WeightSpec((s["dim"], d))
            specs[self.name + "side.proj"] = WeightSpec((d, s["dim"]))
        return specs

    def load_weights(self, tensors):
        if self.gated:
            for q in self._subs():
                self.gates[q] = (tensors["%srg%d" % (self.name, q)],
                                 tensors["%srg%d.b" % (self.name, q)].to(torch.float32).contiguous())
        if self.side:
            self.side_table = tensors[self.side["table"]]
            self.side_gate, self.side_proj = tensors[self.name + "side.gate"], tensors[self.name + "side.proj"]

    def _sublayer(self, q, x, ctx, f, norm_in, norm_out, copy):
        from .linear import linear
        rt = self.runtime
        h = ctx.ws.buffer("normed", tuple(x.shape), rt.dtype)
        norm_in.forward(x, h)
        y = f(h)
        gate = bias = None
        if self.gated:
            w, bias = self.gates[q]
            gate = ctx.ws.buffer("result_gate", tuple(x.shape), rt.dtype)
            linear(h, w, gate, rt.gemm_impl, ws=ctx.ws)
        weight, eps = norm_out.deferred()
        ops.gated_norm_into_stream(y, gate, bias, weight, x, eps, copy=copy)

    def forward(self, x, pending, ctx, cache):
        from .linear import linear
        rt = self.runtime
        if isinstance(pending, StreamCopy):
            pending = None
        if pending is not None:
            ops.residual_add(x, pending[0], pending[1])
        # the token input reads the stream in the compute dtype: the last sublayer's kernel writes that copy along
        copy = None
        if self.side is not None:
            copy = x if rt.dtype == x.dtype else ctx.ws.buffer("stream_copy", tuple(x.shape), rt.dtype)
        has_ffn = self.feed_forward is not None
        last_copy = None if copy is x else copy
        self._sublayer(1, x, ctx, lambda h: self.mixer.forward(h, ctx, cache), self.mixer_norm, self.mixer_out_norm,
                       None if has_ffn else last_copy)
        if has_ffn:
            self._sublayer(2, x, ctx, lambda h: self.feed_forward.forward(h, ctx), self.feed_forward_norm,
                           self.feed_forward_out_norm, last_copy)
        if self.side is not None:
            s, T = self.side, x.shape[0]
            z = ctx.ws.buffer("side_z", (T, s["dim"]), rt.dtype)
            linear(copy, self.side_gate, z, rt.gemm_impl, ws=ctx.ws)
            g = ctx.ws.buffer("side_g", (T, s["dim"]), rt.dtype)
            ops.token_gate(z, self.side_table, ctx.tokens, s["first_column"], g)
            y = ctx.ws.buffer("side_y", tuple(x.shape), rt.dtype)
            linear(g, self.side_proj, y, rt.gemm_impl, ws=ctx.ws)
            weight, eps = self.side_norm.deferred()
            ops.gated_norm_into_stream(y, None, None, weight, x, eps)          # no gate: the plain norm into the stream
        return None
