"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, computed in float32 on the
float32 residual stream (call sites src/models/jiuge/jiuge.cpp:198,246,262;
eps = rms_norm_eps, scripts/jiuge.py:132; weights kept in float32,
scripts/jiuge.py:146,209-215)."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Norm, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, name, runtime, size: int, eps: float, weight_offset: float = 0.0, tensor=None,
                 scale_tensor=None, out_mult: float = 1.0):
        """``weight_offset``: what is added to the stored weight (1.0 for weights stored around zero, y = x r (1 + w));
        the sum is formed once, in float32, when the weights are loaded.  ``tensor``: the weight's full name when it
        is not ``name + "weight"``.  ``scale_tensor``: the full name of a second vector the normed row is multiplied by
        element by element (a layer scale), ``out_mult``: a constant factor on the result (a residual multiplier);
        both join the weight in float32 at load, y = x r (w * s * m), so the kernels see one vector."""
        super().__init__(name, runtime)
        self.size = size
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.tensor = tensor if tensor is not None else name + "weight"
        self.scale_tensor = scale_tensor
        self.out_mult = float(out_mult)
        self.weight = None

    def weight_specs(self):
        specs = {self.tensor: WeightSpec((self.size,), "vector", mean=(1.0 - self.weight_offset) if self.weight_offset else None)}
        if self.scale_tensor is not None:
            specs[self.scale_tensor] = WeightSpec((self.size,), "vector")
        return specs

    def load_weights(self, tensors):
        w = tensors[self.tensor]
        w = (w.to(torch.float32) + self.weight_offset).contiguous() if self.weight_offset else w
        if self.scale_tensor is not None:
            w = w.to(torch.float32) * tensors[self.scale_tensor].to(torch.float32)
        if self.out_mult != 1.0:
            w = w.to(torch.float32) * self.out_mult
        self.weight = w.contiguous()

    def forward_into_stream(self, y, x, copy=None, bias=None):
        """x += norm(y + bias), the norm on a sublayer's output; ``copy`` receives the new x in its dtype."""
        return ops.norm_into_stream(y, self.weight, x, self.eps, bias=bias, copy=copy)

    def forward(self, x, out, rows=None, out_scale: float = 1.0):
        return ops.rmsnorm(x, self.weight, out, self.eps, out_scale, rows)

    def forward_add(self, x, y, alpha, out):
        return ops.add_rmsnorm(x, y, alpha, self.weight, out, self.eps)

    def deferred(self):
        return (self.weight, self.eps)

    def native_desc(self):
        from ..kernels.lib import IcNorm
        w = self.weight
        if not (self._forward_is(RMSNorm) and w is not None and w.is_cuda and w.dtype == torch.float32
                and w.is_contiguous()):
            return None
        return IcNorm(w.data_ptr(), self.eps)
