"""Attention over the last ``window`` tokens plus one mean key and value for every block of ``block`` tokens that lies
wholly before them.  The query at position i sees token j when 0 <= i - j < window, and block b (positions b*block ..
b*block + block - 1) once b*block + block - 1 <= i - window; a token that has left the window while its block is not
yet complete (or not yet wholly outside) is not seen at all.  A block's key is the mean of its keys as the cache holds
them (rotated), its value the mean of its values.  No window: every earlier token, no blocks.

Options, each a parameter:
  * grouped queries, separate key and value sizes per head,
  * rotation of adjacent pairs (2i, 2i+1) of the first ``rot_dims`` entries of queries and keys by position * base^(-2i/rot_dims),
  * weights ``sigmoid``: sigmoid(scale q.k + bias[head]) for tokens and blocks alike, not normalised over the keys
    (``head_bias``: the tensor ``pb``, one number per head).

q, k, v are rows of ONE projection.  One row kernel rotates and writes keys and values into the paged cache; a second
one forms the means of the blocks that the step completes and writes them into pages of their own (one row per block,
never given back, ``CacheNeed.block_rows``); the attention kernels then walk both.  The token cache is a window
group: it keeps max(window, block) tokens, so that a block's tokens are still there when its last one arrives.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import CacheNeed, Mixer, register_part
from .linear import linear


def pair_frequencies(rot_dims: int, base: float) -> torch.Tensor:
    """f_i = base^(-2i/rot_dims), i < rot_dims / 2, as float32 [2, rot_dims / 2]: the float64 value rounded, and what the
    rounding left (the kernel forms the angle from both, so that its error does not grow with the position)."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / rot_dims)
    hi = f.to(torch.float32)
    return torch.stack([hi, (f - hi.double()).to(torch.float32)]).contiguous()


@register_part("mixer", "pooled_attention")
class PooledAttention(Mixer):
    graph_safe = True

    def __init__(self, name, runtime, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
                 score_scale: float, window=None, block=None, rot_dims: int = 0, rot_base=None, weights: str = "sigmoid",
                 head_bias: bool = True):
        super().__init__(name, runtime)
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError("pooled attention: %d heads are not a multiple of %d kv heads" % (num_heads, num_kv_heads))
        if not (0 < key_dim <= 512 and 0 < value_dim <= 512):
            raise ValueError("pooled attention: key and value sizes must lie in 1..512 (got %d, %d)" % (key_dim, value_dim))
        if weights != "sigmoid":
            raise ValueError("pooled attention: weights %r (have sigmoid)" % (weights,))
        rot_dims = int(rot_dims or 0)
        if rot_dims < 0 or rot_dims % 2 or rot_dims > key_dim:
            raise ValueError("pooled attention: rot_dims must be even and at most the key size (got %d)" % rot_dims)
        if rot_dims and not (rot_base and float(rot_base) > 0):
            raise ValueError("pooled attention: a rotation needs a positive base")
        self.hidden_size = int(hidden_size)
        self.nh, self.nkvh, self.dk, self.dv = int(num_heads), int(num_kv_heads), int(key_dim), int(value_dim)
        self.scale = float(score_scale)
        self.window = int(window) if window else 0
        self.block = int(block) if (block and self.window) else 0
        if self.window < 0 or self.block < 0:
            raise ValueError("pooled attention: window and block must not be negative")
        self.rot_dims = rot_dims
        self.freq = pair_frequencies(rot_dims, rot_base).to(runtime.device) if rot_dims else None
        self.head_bias = bool(head_bias)
        self.nq, self.nk, self.nv = self.nh * self.dk, self.nkvh * self.dk, self.nkvh * self.dv
        self.na = self.nh * self.dv
        self.w_rows = self.w_o = self.bias = None

    def cache_need(self):
        # a block's tokens must still be there when its last one arrives: the cache keeps max(window, block) tokens
        keep = max(self.window, self.block) if self.window else None
        return CacheNeed("kv", self.nkvh, self.dk, keep, plane_dims=(self.dk, self.dv), block_rows=self.block)

    # ---- weights ------------------------------------------------------------------------------
    def weight_specs(self):
        n, d = self.name, self.hidden_size
        pack = n + "qkv.packed"
        specs = {
            n + "q": WeightSpec((self.nq, d), pack=(pack, 0)),
            n + "k": WeightSpec((self.nk, d), pack=(pack, 1)),
            n + "v": WeightSpec((self.nv, d), pack=(pack, 2)),
            n + "o": WeightSpec((d, self.na)),
        }
        if self.head_bias:
            specs[n + "pb"] = WeightSpec((self.nh,), "vector", mean=0.0)
        return specs

    def load_weights(self, tensors):
        n = self.name
        packed = tensors.get(n + "qkv.packed")
        if packed is None:
            mats = [tensors[n + s] for s in ("q", "k", "v")]
            if len({m.dtype for m in mats}) > 1:
                mats = [m.to(torch.float32) for m in mats]
            packed = torch.cat(mats, dim=0).contiguous()
        self.w_rows = packed
        self.w_o = tensors[n + "o"]
        self.bias = tensors[n + "pb"].to(torch.float32).contiguous() if self.head_bias else None

    # ---- forward ------------------------------------------------------------------------------
    def forward(self, h, ctx, cache):
        rt = self.runtime
        T = h.shape[0]
        rows = ctx.ws.buffer("pooled_rows", (T, self.w_rows.shape[0]), rt.dtype)
        linear(h, self.w_rows, rows, rt.gemm_impl, ws=ctx.ws)
        q = ctx.ws.buffer("pooled_q", (T, self.nq), rt.dtype)
        ops.rope_pairs_store(rows, ctx.positions, self.freq, self.rot_dims, q, cache.k, cache.v,
                             cache.slots if cache.writes else None, self.nh, self.nkvh, self.dk, self.dv, ctx.page_size)
        blocks = cache.blocks if self.block else None
        if self.block and blocks is None:
            raise RuntimeError("pooled attention %s: the cache holds no rows for the blocks' means" % self.name)
        if blocks is not None and cache.writes:
            ops.pool_blocks(cache.k, cache.v, blocks.k, blocks.v, cache.block_tables, blocks.block_tables, ctx.req_rows,
                            ctx.positions, ctx.R, max(ctx.req_len), self.block, self.nkvh, self.dk, self.dv, ctx.page_size)
        out = ctx.ws.buffer("pooled_out", (T, self.na), rt.dtype)
        self._attend(q, out, ctx, cache, blocks)
        y = ctx.ws.buffer("mixer_out", (T, self.hidden_size), rt.dtype)
        linear(out, self.w_o, y, rt.gemm_impl, ws=ctx.ws)
        return y

    def portion_tile_rows(self):
        return ops.attention_prefill_tile_rows()

    def _attend(self, q, out, ctx, cache, blocks):
        """Single-token rows go to the split kernel, prompt portions to the matrix-core kernel, where the sizes have one (and
        the runtime does not ask for the general kernel alone); everything else to the general kernel."""
        rt = self.runtime
        planes = (cache.k, cache.v, blocks.k if blocks else None, blocks.v if blocks else None, cache.block_tables,
                  blocks.block_tables if blocks else None)
        tail = (self.bias, self.nh, self.nkvh, self.dk, self.dv, ctx.page_size, self.scale, self.window, self.block)
        n_dec, n_tiles = ctx.n_decode_rows, ctx.n_prefill_tiles
        tiled = rt.attention_impl == "auto" and n_dec + n_tiles > 0
        use_dec = tiled and n_dec > 0 and ops.attention_pooled_decode_supported(rt.dtype, self.dk, self.dv)
        use_pre = tiled and n_tiles > 0 and ops.attention_pooled_prefill_supported(rt.dtype, self.dk, self.dv, ctx.page_size)
        if not tiled or not (use_dec or n_dec == 0) or not (use_pre or n_tiles == 0):
            ops.attention_pooled_generic(q, out, *planes, ctx.token_req, ctx.positions, *tail)
            return
        if use_dec:
            n_split = self._splits(ctx)
            parts = ctx.ws.buffer("pooled_parts", (n_split * n_dec * self.nh * self.dv,), torch.float32) if n_split > 1 else None
            ops.attention_pooled_decode(q, out, *planes, None if ctx.decode_rows_identity else ctx.decode_rows, n_dec,
                                        ctx.token_req, ctx.positions, parts, *tail, n_split=n_split)
        if use_pre:
            ops.attention_pooled_prefill(q, out, *planes, ctx.prefill_tiles, n_tiles, *tail)

    def _splits(self, ctx) -> int:
        """Ways to split what single-token rows see: enough blocks of threads to fill the chip about four times, none with fewer
        than 64 items; from the number of rows and the step's rounded key count, so that recorded steps split as eager ones."""
        if ctx.fixed_decode_splits is not None:
            return max(1, min(32, ctx.fixed_decode_splits))
        most = ctx.max_context or 1
        if self.window:
            most = min(most, self.window) + (most // self.block if self.block else 0)
        want = -(-4 * ctx.cu_count // max(1, ctx.n_decode_rows * self.nkvh))
        return max(1, min(32, want, most // 64))
