"""Mixers that carry a fixed-size float32 state per sequence instead of a cache of keys.

``rglru``: a gated diagonal linear recurrence between two branches of ``width`` channels.  With h the normed input,
    y = gelu_tanh(W_y h + b_y),   u = conv(W_x h + b_x)            (a causal convolution per channel, no activation)
    r = sigmoid(A_b u_b + a_b),   i = sigmoid(I_b u_b + i_b)       (u cut into ``blocks`` parts, a square matrix each)
    log a = -8 r softplus(lam),   S_t = a S_(t-1) + sqrt(1 - a^2) i u,   out = W_o (S y).
``mamba2``: a state-space recurrence with a matrix state [N, P] per head.  W_in h = [z | x | B | C | dt]; x, B, C pass
    a causal convolution per channel and silu; dt = softplus(dt + dt_bias);
    S_t = exp(-exp(A_log) dt) S_(t-1) + dt B x^T,   y = S^T C + D x;   out = W_o (rms_in_groups(y silu(z)) * w).
``decay_linear_attention``: linear attention with a fixed decay per head and a matrix state [dim, vdim] per head.
    q = silu(W_q h), k = silu(W_k h), v = silu(W_v h);   S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t;
    out = W_o (rms(o) * w * sigmoid(W_g h))    (the norm over all heads together, the gate after it).
The first two keep, beside the recurrent state, the convolution's last taps - 1 inputs; one float32 vector per request holds
the two.  The state starts at zero.  Products run in the compute dtype; gates, decays, step sizes and the state are float32.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import CacheNeed, Mixer, register_part
from .linear import linear


CHUNK_SCRATCH_BYTES = 256 << 20     # most scratch memory the chunks' states of one recurrence may take


def chunk_plan(ctx, n_state: int, n_factors: int, name: str):
    """How a step's recurrence is cut into chunks that run side by side: None for a step of few tokens per request
    (one pass from and to the state), else (chunk_len, max_chunks, scratch, scratch) with up to 32 chunks of at least 32
    tokens for the longest portion, fewer where the chunks' states would not fit the scratch memory."""
    longest = max(ctx.req_len) if ctx.req_len else 1
    if longest < 64:
        return None
    most = max(1, min(32, longest // 32, CHUNK_SCRATCH_BYTES // (4 * n_state * ctx.R)))
    if most <= 1:
        return None
    chunk_len = (longest + most - 1) // most
    max_chunks = (longest + chunk_len - 1) // chunk_len
    return (chunk_len, max_chunks, ctx.ws.buffer(name + "_chunk_states", (ctx.R * max_chunks * n_state,), torch.float32),
            ctx.ws.buffer(name + "_chunk_factors", (ctx.R * max_chunks * n_factors,), torch.float32))


@register_part("mixer", "rglru")
class GatedLinearRecurrence(Mixer):
    graph_safe = True

    def __init__(self, name, runtime, hidden_size: int, width: int, blocks: int, conv_taps: int, decay_scale: float = 8.0):
        super().__init__(name, runtime)
        if width <= 0 or blocks <= 0 or width % blocks:
            raise ValueError("rglru: width %d is not a multiple of %d blocks" % (width, blocks))
        if not 1 <= conv_taps <= 8:
            raise ValueError("rglru: 1..8 convolution taps (got %d)" % conv_taps)
        self.hidden_size, self.width, self.blocks, self.taps = int(hidden_size), int(width), int(blocks), int(conv_taps)
        self.bw = self.width // self.blocks
        self.decay_scale = float(decay_scale)
        self.conv_offset = self.width                      # the state: [S: width | conv inputs: (taps - 1) * width]
        self.state_size = self.width * self.taps

    def cache_need(self):
        return CacheNeed("state", state_shape=(self.state_size,), state_dtype=torch.float32)

    def weight_specs(self):
        n, d, w, b, bw = self.name, self.hidden_size, self.width, self.blocks, self.bw
        pack = n + "yx.packed"
        return {
            n + "y": WeightSpec((w, d), pack=(pack, 0)), n + "x": WeightSpec((w, d), pack=(pack, 1)),
            n + "y.b": WeightSpec((w,), "vector", mean=0.0), n + "x.b": WeightSpec((w,), "vector", mean=0.0),
            n + "conv": WeightSpec((w, self.taps), "vector", mean=1.0 / self.taps), n + "conv.b": WeightSpec((w,), "vector", mean=0.0),
            n + "ra": WeightSpec((b, bw, bw)), n + "ri": WeightSpec((b, bw, bw)),
            n + "ra.b": WeightSpec((b, bw), "vector", mean=0.0), n + "ri.b": WeightSpec((b, bw), "vector", mean=0.0),
            n + "lam": WeightSpec((w,), "vector", mean=0.0),
            n + "o": WeightSpec((d, w)),
        }

    def load_weights(self, tensors):
        n = self.name
        packed = tensors.get(n + "yx.packed")
        if packed is None:
            packed = torch.cat([tensors[n + "y"], tensors[n + "x"]], dim=0).contiguous()
        self.w_yx = packed
        self.b_y, self.b_x = tensors[n + "y.b"], tensors[n + "x.b"]
        self.conv_w, self.conv_b = tensors[n + "conv"].contiguous(), tensors[n + "conv.b"]
        # the two gate matrices of a block one after the other: [blocks, 2 bw, bw], biases alike
        self.w_gate = torch.cat([tensors[n + "ra"], tensors[n + "ri"]], dim=1).contiguous()
        self.b_gate = torch.cat([tensors[n + "ra.b"], tensors[n + "ri.b"]], dim=1).to(torch.float32).contiguous().view(-1)
        lam = tensors[n + "lam"].to(torch.float64)
        self.decay = (-self.decay_scale * torch.nn.functional.softplus(lam)).to(torch.float32).contiguous()
        self.w_o = tensors[n + "o"]

    def forward(self, h, ctx, cache):
        rt, T, w = self.runtime, h.shape[0], self.width
        yx = ctx.ws.buffer("rglru_yx", (T, 2 * w), rt.dtype)
        linear(h, self.w_yx, yx, rt.gemm_impl, ws=ctx.ws)
        u = ctx.ws.buffer("rglru_u", (T, w), torch.float32)
        u_c = None if rt.dtype == torch.float32 else ctx.ws.buffer("rglru_u_copy", (T, w), rt.dtype)
        lists = (ctx.req_rows, ctx.state_slots, ctx.R)
        ops.causal_conv(yx[:, w:], self.conv_w, self.conv_b, u, cache.state, self.conv_offset, ctx.token_req, *lists,
                        in_bias=self.b_x, out_copy=u_c)
        gates = ctx.ws.buffer("rglru_gates", (T, 2 * w), torch.float32)
        ops.blocked_product((u if u_c is None else u_c).view(T, self.blocks, self.bw), self.w_gate,
                            gates.view(T, self.blocks, 2 * self.bw))
        out = ctx.ws.buffer("rglru_out", (T, w), rt.dtype)
        ops.rglru_scan(gates, self.b_gate, u, yx[:, :w], self.b_y, self.decay, self.bw, out, cache.state, 0, *lists,
                       chunks=chunk_plan(ctx, w, w, "rglru"))
        y = ctx.ws.buffer("mixer_out", (T, self.hidden_size), rt.dtype)
        linear(out, self.w_o, y, rt.gemm_impl, ws=ctx.ws)
        return y


@register_part("mixer", "mamba2")
class StateSpaceMixer(Mixer):
    graph_safe = True

    def __init__(self, name, runtime, hidden_size: int, heads: int, head_dim: int, state_dim: int, groups: int,
                 conv_taps: int, norm_groups: int, norm_eps: float):
        super().__init__(name, runtime)
        if heads <= 0 or groups <= 0 or heads % groups:
            raise ValueError("mamba2: %d heads are not a multiple of %d groups" % (heads, groups))
        if not 0 < head_dim <= 256:
            raise ValueError("mamba2: a head's size must lie in 1..256 (got %d)" % head_dim)
        if state_dim <= 0 or 2 * state_dim + head_dim > 1024 or -(-state_dim // (256 // head_dim)) > 128:
            raise ValueError("mamba2: a head's state of %d x %d is beyond what the kernel keeps in registers" % (state_dim, head_dim))
        self.inner = heads * head_dim
        if norm_groups <= 0 or self.inner % norm_groups:
            raise ValueError("mamba2: %d columns are not a multiple of %d norm groups" % (self.inner, norm_groups))
        if not 1 <= conv_taps <= 8:
            raise ValueError("mamba2: 1..8 convolution taps (got %d)" % conv_taps)
        self.hidden_size, self.heads, self.P, self.N, self.G = int(hidden_size), int(heads), int(head_dim), int(state_dim), int(groups)
        self.taps, self.norm_groups, self.eps = int(conv_taps), int(norm_groups), float(norm_eps)
        self.channels = self.inner + 2 * self.G * self.N             # what passes the convolution: x, B, C
        self.proj = 2 * self.inner + 2 * self.G * self.N + self.heads
        self.conv_offset = self.inner * self.N                       # the state: [S: heads N P | conv inputs: (taps - 1) * channels]
        self.state_size = self.conv_offset + (self.taps - 1) * self.channels

    def cache_need(self):
        return CacheNeed("state", state_shape=(self.state_size,), state_dtype=torch.float32)

    def weight_specs(self):
        n, d = self.name, self.hidden_size
        return {
            n + "in": WeightSpec((self.proj, d)),
            n + "conv": WeightSpec((self.channels, self.taps), "vector", mean=1.0 / self.taps),
            n + "conv.b": WeightSpec((self.channels,), "vector", mean=0.0),
            n + "dt_bias": WeightSpec((self.heads,), "vector", mean=0.0),
            n + "A_log": WeightSpec((self.heads,), "vector", mean=0.0),
            n + "D": WeightSpec((self.heads,), "vector"),
            n + "norm": WeightSpec((self.inner,), "vector"),
            n + "o": WeightSpec((d, self.inner)),
        }

    def load_weights(self, tensors):
        n = self.name
        self.w_in, self.w_o = tensors[n + "in"], tensors[n + "o"]
        self.conv_w, self.conv_b = tensors[n + "conv"].contiguous(), tensors[n + "conv.b"]
        self.dt_bias, self.d_skip, self.norm_w = tensors[n + "dt_bias"], tensors[n + "D"], tensors[n + "norm"]
        self.neg_a = (-torch.exp(tensors[n + "A_log"].to(torch.float64))).to(torch.float32).contiguous()

    def forward(self, h, ctx, cache):
        rt, T, inner, ch = self.runtime, h.shape[0], self.inner, self.channels
        proj = ctx.ws.buffer("ssm_proj", (T, self.proj), rt.dtype)
        linear(h, self.w_in, proj, rt.gemm_impl, ws=ctx.ws)
        lists = (ctx.req_rows, ctx.state_slots, ctx.R)
        xbc = ctx.ws.buffer("ssm_xbc", (T, ch), torch.float32)
        ops.causal_conv(proj[:, inner:inner + ch], self.conv_w, self.conv_b, xbc, cache.state, self.conv_offset,
                        ctx.token_req, *lists, act="silu")
        y = ctx.ws.buffer("ssm_y", (T, inner), torch.float32)
        ops.ssm_scan(xbc, proj[:, inner + ch:], self.dt_bias, self.neg_a, self.d_skip, self.heads, self.P, self.N, self.G, y,
                     cache.state, 0, *lists, chunks=chunk_plan(ctx, inner * self.N, self.heads, "ssm"))
        g = ctx.ws.buffer("ssm_gated", (T, inner), rt.dtype)
        ops.gated_group_norm(y, proj[:, :inner], self.norm_w, self.norm_groups, self.eps, g)
        out = ctx.ws.buffer("mixer_out", (T, self.hidden_size), rt.dtype)
        linear(g, self.w_o, out, rt.gemm_impl, ws=ctx.ws)
        return out


@register_part("mixer", "decay_linear_attention")
class DecayLinearAttention(Mixer):
    """Linear attention whose state decays by a fixed factor per head.  The recurrence is the state-space one with keys
    for B, values for x, queries for C, one group per head, steps of one and no skip term, so it runs in the same scan
    kernel (single pass for few tokens, chunks side by side for prompt portions), which reads q, k, v straight from the
    projection's rows and applies their silu on the way in.  The four matrices are one projection, laid out [v | k | q | g]."""
    graph_safe = True

    def __init__(self, name, runtime, hidden_size: int, heads: int, key_dim: int, value_dim: int, decay, norm_eps: float):
        super().__init__(name, runtime)
        decay = [float(a) for a in decay]
        if heads <= 0 or len(decay) != heads:
            raise ValueError("linear attention: %d heads but %d decays" % (heads, len(decay)))
        if any(not 0.0 <= a <= 1.0 for a in decay):
            raise ValueError("linear attention: a decay lies outside [0, 1]")
        if not 0 < value_dim <= 256:
            raise ValueError("linear attention: a head's value size must lie in 1..256 (got %d)" % value_dim)
        if key_dim <= 0 or 2 * key_dim + value_dim > 1024 or -(-key_dim // (256 // value_dim)) > 128:
            raise ValueError("linear attention: a head's state of %d x %d is beyond what the kernel keeps in registers" % (key_dim, value_dim))
        self.hidden_size, self.heads, self.dk, self.dv = int(hidden_size), int(heads), int(key_dim), int(value_dim)
        self.eps = float(norm_eps)
        self.nq, self.nv = self.heads * self.dk, self.heads * self.dv
        self.proj = 2 * self.nq + 2 * self.nv
        self.state_size = self.heads * self.dk * self.dv
        self.decay = torch.tensor(decay, dtype=torch.float64).to(torch.float32).to(runtime.device)

    def cache_need(self):
        return CacheNeed("state", state_shape=(self.state_size,), state_dtype=torch.float32)

    def weight_specs(self):
        n, d = self.name, self.hidden_size
        pack = n + "vkqg.packed"
        return {
            n + "v": WeightSpec((self.nv, d), pack=(pack, 0)), n + "k": WeightSpec((self.nq, d), pack=(pack, 1)),
            n + "q": WeightSpec((self.nq, d), pack=(pack, 2)), n + "g": WeightSpec((self.nv, d), pack=(pack, 3)),
            n + "norm": WeightSpec((self.nv,), "vector"),
            n + "o": WeightSpec((d, self.nv)),
        }

    def load_weights(self, tensors):
        n = self.name
        packed = tensors.get(n + "vkqg.packed")
        if packed is None:
            mats = [tensors[n + s] for s in ("v", "k", "q", "g")]
            if len({m.dtype for m in mats}) > 1:
                mats = [m.to(torch.float32) for m in mats]
            packed = torch.cat(mats, dim=0).contiguous()
        self.w_rows, self.w_o, self.norm_w = packed, tensors[n + "o"], tensors[n + "norm"]

    def forward(self, h, ctx, cache):
        rt, T = self.runtime, h.shape[0]
        rows = ctx.ws.buffer("linattn_rows", (T, self.proj), rt.dtype)
        linear(h, self.w_rows, rows, rt.gemm_impl, ws=ctx.ws)
        o = ctx.ws.buffer("linattn_o", (T, self.nv), torch.float32)
        ops.ssm_scan(rows, None, None, self.decay, None, self.heads, self.dv, self.dk, self.heads, o, cache.state, 0,
                     ctx.req_rows, ctx.state_slots, ctx.R, chunks=chunk_plan(ctx, self.state_size, self.heads, "linattn"),
                     in_act="silu")
        g = ctx.ws.buffer("linattn_gated", (T, self.nv), rt.dtype)
        ops.gated_group_norm(o, rows[:, self.nv + 2 * self.nq:], self.norm_w, 1, self.eps, g, gate_after=True)
        out = ctx.ws.buffer("mixer_out", (T, self.hidden_size), rt.dtype)
        linear(g, self.w_o, out, rt.gemm_impl, ws=ctx.ws)
        return out
