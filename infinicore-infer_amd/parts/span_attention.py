"""Softmax attention whose keys and values may differ in size per head and whose queries see a span of the
keys: the last ``window`` keys plus the first ``keep_first`` keys of the sequence (query i sees key j when
j <= i and (i - j < window or j < keep_first); no window: every earlier key).  Positions do not enter the
scores.  Options, each a parameter:

  * biases on the q, k, v projections and on the output projection,
  * a norm on queries and keys to unit root mean square, per head (one weight of the key size, shared by the
    heads, or no weight at all) or over the whole projection before it is cut into heads (a weight of the
    projection's size),
  * a cap on the scaled score, s <- c tanh(s / c),
  * a sink: one more term in the softmax's denominator that has no value, p_j = e^{s_j} / (e^{z} + sum e^{s_j}),
    with z = 0 or z a learned number per head (the tensor ``sink``), neither scaled nor capped,
  * value mixing: the first mixing layer of the model keeps its values of the step's tokens, every later one
    replaces its own by (1 - lambda) v + lambda v_first before they are cached (lambda a learned scalar),
  * an output gate: the concatenated heads are multiplied by sigmoid(W_g h) before the output projection.

q, k, v and the gate are rows of ONE projection; a single row kernel then adds the biases, applies the norms,
mixes the values, and writes keys and values into the paged cache (K and V planes of different widths).  The
scores never reach memory: the attention kernels walk the cache with a float32 running softmax.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import CacheNeed, Mixer, register_part
from .linear import linear

_NORM_MODES = {None: 0, "none": 0, "head": 1, "row": 2}
_MIX_MODES = {None: 0, "none": 0, "keep": 1, "mix": 2}


@register_part("mixer", "span_attention")
class SpanAttention(Mixer):
    graph_safe = True
    defers_bias = True           # forward(.., defer_bias=True) leaves the output projection's bias to the caller

    def __init__(self, name, runtime, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int,
                 value_dim: int, softmax_scale: float, window=None, keep_first: int = 0, sink: bool = False,
                 qk_norm=None, qk_norm_eps: float = 1e-6, qkv_bias: bool = False, out_bias: bool = False,
                 gate: bool = False, value_mix=None, value_mix_width=None, value_mix_optional: bool = False,
                 softcap=None, qk_norm_weight: bool = True):
        """``sink``: False, True (the constant term exp(0)) or "learned" (one number per head, the tensor ``sink``).
        ``softcap``: None or the cap c > 0.  ``qk_norm_weight`` False: the per-head norm has no weight tensors.
        ``qk_norm``: None, "head" or "row".  ``value_mix``: None, "keep" (this layer's values are the ones later
        layers mix in) or "mix"; all mixing layers of a model have the same kv heads and value size.
        ``value_mix_optional``: the files may hold the mixing scalar although this layer does not mix."""
        super().__init__(name, runtime)
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError("span attention: %d heads are not a multiple of %d kv heads" % (num_heads, num_kv_heads))
        if not (0 < key_dim <= 512 and 0 < value_dim <= 512):
            raise ValueError("span attention: key and value sizes must lie in 1..512 (got %d, %d)" % (key_dim, value_dim))
        if qk_norm not in _NORM_MODES or value_mix not in _MIX_MODES:
            raise ValueError("span attention: qk_norm %r / value_mix %r unknown" % (qk_norm, value_mix))
        self.hidden_size = hidden_size
        self.nh, self.nkvh, self.dk, self.dv = num_heads, num_kv_heads, key_dim, value_dim
        self.scale = float(softmax_scale)
        self.window = int(window) if window else 0
        self.keep_first = int(keep_first or 0) if self.window else 0
        if self.keep_first < 0:
            raise ValueError("span attention: keep_first must not be negative")
        if sink not in (False, True, None, "learned"):
            raise ValueError("span attention: sink is False, True or 'learned' (got %r)" % (sink,))
        self.sink = bool(sink)
        self.sink_learned = sink == "learned"
        self.softcap = float(softcap) if softcap else 0.0
        if self.softcap < 0:
            raise ValueError("span attention: the score cap must be positive")
        self.norm_weight = bool(qk_norm_weight)
        if not self.norm_weight and qk_norm == "row":
            raise ValueError("span attention: the norm over the whole projection comes with a weight")
        self.sinks = None
        self.norm_mode = _NORM_MODES[qk_norm]
        self.qk_norm_eps = float(qk_norm_eps)
        self.qkv_bias, self.out_bias, self.gate = bool(qkv_bias), bool(out_bias), bool(gate)
        self.mix_mode = _MIX_MODES[value_mix]
        self.mix_optional = bool(value_mix_optional)
        self.nq, self.nk, self.nv = self.nh * self.dk, self.nkvh * self.dk, self.nkvh * self.dv
        self.na = self.nh * self.dv                       # width of the concatenated heads
        self.w_rows = self.w_o = self.b_rows = self.b_o = self.q_norm = self.k_norm = self.mix_lambda = None

    def cache_need(self):
        return CacheNeed("kv", self.nkvh, self.dk, self.window or None, plane_dims=(self.dk, self.dv),
                         keep_first=self.keep_first)

    def portion_tile_rows(self):
        return ops.attention_prefill_tile_rows()

    # ---- weights ------------------------------------------------------------------------------
    def weight_specs(self):
        n, d = self.name, self.hidden_size
        pack, bpack = n + "qkvg.packed", n + "qkv_bias.packed"
        specs = {
            n + "q": WeightSpec((self.nq, d), pack=(pack, 0)),
            n + "k": WeightSpec((self.nk, d), pack=(pack, 1)),
            n + "v": WeightSpec((self.nv, d), pack=(pack, 2)),
            n + "o": WeightSpec((d, self.na)),
        }
        if self.gate:
            specs[n + "g"] = WeightSpec((self.na, d), pack=(pack, 3))
        if self.qkv_bias:
            specs[n + "q.b"] = WeightSpec((self.nq,), "vector", pack=(bpack, 0), mean=0.0)
            specs[n + "k.b"] = WeightSpec((self.nk,), "vector", pack=(bpack, 1), mean=0.0)
            specs[n + "v.b"] = WeightSpec((self.nv,), "vector", pack=(bpack, 2), mean=0.0)
        if self.out_bias:
            specs[n + "o.b"] = WeightSpec((d,), "vector", mean=0.0)
        if self.sink_learned:
            specs[n + "sink"] = WeightSpec((self.nh,), "vector", mean=0.0)
        if self.norm_mode and self.norm_weight:
            per_head = self.norm_mode == 1
            specs[n + "q.norm"] = WeightSpec((self.dk if per_head else self.nq,), "vector")
            specs[n + "k.norm"] = WeightSpec((self.dk if per_head else self.nk,), "vector")
        if self.mix_mode or self.mix_optional:
            # the keeping layer holds a scalar too, which nothing reads
            specs[n + "vmix"] = WeightSpec((), "vector", optional=self.mix_mode == 0, mean=0.5)
        return specs

    def load_weights(self, tensors):
        n = self.name
        names = ["q", "k", "v"] + (["g"] if self.gate else [])
        packed = tensors.get(n + "qkvg.packed")
        if packed is None:
            mats = [tensors[n + s] for s in names]
            if len({m.dtype for m in mats}) > 1:
                mats = [m.to(torch.float32) for m in mats]
            packed = torch.cat(mats, dim=0).contiguous()
        self.w_rows = packed
        self.w_o = tensors[n + "o"]
        if self.qkv_bias:
            b = tensors.get(n + "qkv_bias.packed")
            if b is None:
                b = torch.cat([tensors[n + s + ".b"].to(torch.float32).reshape(-1) for s in ("q", "k", "v")]).contiguous()
            self.b_rows = b
        self.b_o = tensors[n + "o.b"] if self.out_bias else None
        if self.norm_mode and self.norm_weight:
            self.q_norm, self.k_norm = tensors[n + "q.norm"], tensors[n + "k.norm"]
        if self.sink_learned:
            self.sinks = tensors[n + "sink"].to(torch.float32).contiguous()
        if self.mix_mode == 2:
            self.mix_lambda = tensors[n + "vmix"].reshape(1)

    def deferred_bias(self):
        return self.b_o

    # ---- forward ------------------------------------------------------------------------------
    def forward(self, h, ctx, cache, defer_bias: bool = False):
        rt = self.runtime
        T = h.shape[0]
        rows = ctx.ws.buffer("span_rows", (T, self.w_rows.shape[0]), rt.dtype)
        linear(h, self.w_rows, rows, rt.gemm_impl, ws=ctx.ws)
        q = ctx.ws.buffer("span_q", (T, self.nq), rt.dtype)
        v_keep = ctx.ws.buffer("value_mix_keep", (T, self.nv), torch.float32) if self.mix_mode else None
        ops.qk_norm_store(rows, self.b_rows, self.q_norm, self.k_norm, self.norm_mode, self.qk_norm_eps, self.mix_mode,
                          self.mix_lambda, v_keep, q, cache.k, cache.v, cache.slots if cache.writes else None,
                          self.nh, self.nkvh, self.dk, self.dv, ctx.page_size)
        out = ctx.ws.buffer("span_out", (T, self.na), rt.dtype)
        gate = rows[:, self.nq + self.nk + self.nv:] if self.gate else None
        self._attend(q, out, gate, ctx, cache)
        y = ctx.ws.buffer("mixer_out", (T, self.hidden_size), rt.dtype)
        linear(out, self.w_o, y, rt.gemm_impl, ws=ctx.ws)
        if self.b_o is not None and not defer_bias:
            y.add_(self.b_o.to(y.dtype))
        return y

    def _attend(self, q, out, gate, ctx, cache):
        """Single-token rows go to the split-key kernel, prompt portions to the matrix-core kernel, where the sizes
        have one (and the runtime does not ask for the general kernel alone); everything else to the general kernel."""
        rt = self.runtime
        args = (self.nh, self.nkvh, self.dk, self.dv, ctx.page_size, self.scale, self.window, self.keep_first,
                self.sinks if self.sink_learned else self.sink, self.softcap)
        n_dec, n_tiles = ctx.n_decode_rows, ctx.n_prefill_tiles
        tiled = rt.attention_impl == "auto" and n_dec + n_tiles > 0
        use_dec = tiled and n_dec > 0 and ops.attention_span_decode_supported(rt.dtype, self.dk, self.dv)
        use_pre = (tiled and n_tiles > 0 and self.scale > 0 and ctx.page_size & (ctx.page_size - 1) == 0
                   and ops.attention_span_prefill_supported(rt.dtype, self.dk, self.dv))
        if not (use_dec or n_dec == 0) or not (use_pre or n_tiles == 0) or not tiled:
            ops.attention_span_generic(q, out, gate, cache.k, cache.v, cache.block_tables, ctx.token_req, ctx.positions, *args)
            return
        if use_dec:
            n_split = self._key_splits(ctx)
            part_acc = part_ml = None
            if n_split > 1:
                part_acc = ctx.ws.buffer("span_part_acc", (n_dec * self.nh * n_split * self.dv,), torch.float32)
                part_ml = ctx.ws.buffer("span_part_ml", (n_dec * self.nh * n_split * 2,), torch.float32)
            ops.attention_span_decode(q, out, gate, cache.k, cache.v, cache.block_tables,
                                      None if ctx.decode_rows_identity else ctx.decode_rows, n_dec, ctx.token_req,
                                      ctx.positions, part_acc, part_ml, *args, n_split=n_split)
        if use_pre:
            ops.attention_span_prefill(q, out, gate, cache.k, cache.v, cache.block_tables, ctx.prefill_tiles, n_tiles, *args)

    def _key_splits(self, ctx) -> int:
        """Ways to split the visible keys of single-token rows: the kernel library's rule, from the number of rows and
        the most keys a row can see (the step's rounded key count, or the window with its kept keys when smaller)."""
        if ctx.fixed_decode_splits is not None:
            return max(1, min(32, ctx.fixed_decode_splits))
        most = ctx.max_context or 1
        if self.window:
            most = min(most, self.window + self.keep_first)
        return ops.attention_span_decode_splits(ctx.n_decode_rows, self.nkvh, most, ctx.cu_count)
