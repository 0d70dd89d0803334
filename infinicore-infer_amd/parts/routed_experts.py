"""A feed-forward of routed experts: ``experts`` small gated units W_down (silu(W_gate h) * (W_up h)), of which every
token uses the ``top`` with the largest router scores, plus an optional shared unit of the same form that every token
passes through.

  z = W_router h (float32);  s = sigmoid(z) (``scores="sigmoid"``) or softmax(z) over the experts (``"softmax"``)
  the chosen experts' weights are their scores, renormalised over the chosen ones only with ``renormalize``
  ``weight_on="input"``:  y = sum_chosen expert_e(s_e h);   ``"output"``:  y = sum_chosen s_e expert_e(h)
  y += shared(h)

Tensors: ``router`` [experts, d], ``e<j>.gate`` / ``.up`` [ff, d], ``e<j>.down`` [d, ff], ``shared.gate`` / ``.up`` /
``.down``.  The loader lays all experts' gate and up matrices out as one tensor [experts, 2 ff, d] and the down matrices as
[experts, d, ff].

A step's (token, choice) pairs are sorted by expert on the device (stable).  For few rows every expert's chunk of rows
streams that expert's matrices once (``ops.moe_expert_product``, the gated unit in the first product's epilogue): no
integer leaves the device, so decode steps can be recorded.  For many rows the host reads the experts' row counts and
runs one library product per expert and matrix over its run of rows.
"""
import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import FeedForward, build_part, register_part
from .linear import linear

FEW_ROWS = 64          # up to this many tokens a step the experts' products run without the host seeing the routing


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, name, runtime, hidden_size: int, experts: int, top: int, expert_size: int, shared_size=None,
                 scores: str = "sigmoid", renormalize: bool = False, weight_on: str = "input"):
        super().__init__(name, runtime)
        if not (0 < top <= experts <= 1024 and top <= 16):
            raise ValueError("routed experts: 0 < top <= experts, at most 16 of at most 1024 (got %d of %d)" % (top, experts))
        if scores not in ("sigmoid", "softmax") or weight_on not in ("input", "output"):
            raise ValueError("routed experts: scores %r / weight_on %r unknown" % (scores, weight_on))
        if expert_size <= 0:
            raise ValueError("routed experts: an expert's size must be positive")
        self.hidden_size, self.E, self.top, self.ff = int(hidden_size), int(experts), int(top), int(expert_size)
        self.scores, self.renormalize, self.weight_on = scores, bool(renormalize), weight_on
        self.shared = None
        if shared_size:
            self.shared = build_part("feed_forward", PartSpec("swiglu", name + "shared.", {
                "hidden_size": hidden_size, "intermediate_size": int(shared_size), "gate_name": "gate", "up_name": "up",
                "down_name": "down"}), runtime)
        self.w_router = self.w_gate_up = self.w_down = None

    def sub_parts(self):
        return (self.shared,) if self.shared is not None else ()

    def weight_specs(self):
        n, d, ff = self.name, self.hidden_size, self.ff
        specs = {n + "router": WeightSpec((self.E, d))}
        for e in range(self.E):
            specs["%se%d.gate" % (n, e)] = WeightSpec((ff, d), pack=(n + "experts_gate_up.packed", 2 * e))
            specs["%se%d.up" % (n, e)] = WeightSpec((ff, d), pack=(n + "experts_gate_up.packed", 2 * e + 1))
            specs["%se%d.down" % (n, e)] = WeightSpec((d, ff), pack=(n + "experts_down.packed", e))
        return specs

    def load_weights(self, tensors):
        n, d, ff = self.name, self.hidden_size, self.ff
        self.w_router = tensors[n + "router"]
        gu, dn = tensors.get(n + "experts_gate_up.packed"), tensors.get(n + "experts_down.packed")
        if gu is None:
            gu = torch.cat([tensors["%se%d.%s" % (n, e, s)] for e in range(self.E) for s in ("gate", "up")], dim=0).contiguous()
        if dn is None:
            dn = torch.cat([tensors["%se%d.down" % (n, e)] for e in range(self.E)], dim=0).contiguous()
        self.w_gate_up = gu.view(self.E, 2 * ff, d)
        self.w_down = dn.view(self.E, d, ff)

    def forward(self, h, ctx):
        rt, E, top, d, ff = self.runtime, self.E, self.top, self.hidden_size, self.ff
        T = h.shape[0]
        n = T * top
        buf = ctx.ws.buffer
        logits = buf("moe_logits", (T, E), torch.float32)
        linear(h, self.w_router, logits, rt.gemm_impl, ws=ctx.ws)             # float32 sums of the rows as they are
        ids, weights = buf("moe_ids", (T, top), torch.int32), buf("moe_weights", (T, top), torch.float32)
        ops.moe_route(logits, top, ids, weights, self.scores, self.renormalize)
        offsets, order, place = buf("moe_offsets", (E + 1,), torch.int32), buf("moe_order", (n,), torch.int32), buf("moe_place", (n,), torch.int32)
        ops.moe_sort(ids, E, offsets, order, place)
        on_input = self.weight_on == "input"
        rows = buf("moe_rows", (n, d), rt.dtype)
        ops.moe_gather(h, order, weights.view(-1) if on_input else None, top, rows)
        act, y = buf("moe_act", (n, ff), rt.dtype), buf("moe_y", (n, d), rt.dtype)
        if T <= FEW_ROWS:
            ops.moe_expert_product(rows, self.w_gate_up, offsets, act, glu=True, compute_units=ctx.cu_count)
            ops.moe_expert_product(act, self.w_down, offsets, y, glu=False, compute_units=ctx.cu_count)
        else:
            gate_up = buf("moe_gate_up", (n, 2 * ff), rt.dtype)
            bounds = offsets.tolist()                                          # the host waits for the routing here
            runs = [(e, bounds[e], bounds[e + 1]) for e in range(E) if bounds[e + 1] > bounds[e]]
            for e, a, b in runs:
                linear(rows[a:b], self.w_gate_up[e], gate_up[a:b], rt.gemm_impl, ws=ctx.ws)
            ops.swiglu(gate_up, act)
            for e, a, b in runs:
                linear(act[a:b], self.w_down[e], y[a:b], rt.gemm_impl, ws=ctx.ws)
        shared = self.shared.forward(h, ctx) if self.shared is not None else None
        out = buf("moe_out", (T, d), rt.dtype)
        ops.moe_combine(y, place, None if on_input else weights.view(-1), shared, top, out)
        return out
