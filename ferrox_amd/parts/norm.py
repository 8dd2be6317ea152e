"""RMSNorm (ferrox-core/src/matmul.rs:62-69): y = x * rsqrt(mean(x^2) + eps) * w,
statistics in float32, read from the float32 residual stream.  A design may store
its weight around zero (y = ... * (offset + w)), or have none at all."""
from __future__ import annotations

from .. import ops
from .base import NORMS, Norm, ParamSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    kernel_libraries = ("elementwise",)

    def __init__(self, size: int, eps: float, name: str = "weight", offset: float = 0.0, weight: bool = True,
                 gain: float = 1.0):
        """`name`: what the weight is called behind the part's prefix.  `offset`: the stored tensor is the weight
        minus this number (a weight stored around zero has offset 1); the sum is made once, in float32, and kept in
        float32, so that nothing of the stored tensor's precision is lost.  `weight` False: no tensor, rows are
        brought to unit root mean square and no more.  `gain`: a constant that the normed rows are multiplied by (a
        model that scales its logits by a constant scales the rows in front of its head: the head is linear); it is
        folded into the float32 weight."""
        self.size = int(size)
        self.eps = float(eps)
        self.name = name
        self.offset, self.gain = float(offset), float(gain)
        if not weight and gain != 1.0:
            raise ValueError("a norm without a weight has no gain")
        self.has_weight = bool(weight)
        self.weight = None

    def param_specs(self):
        if not self.has_weight:
            return {}
        return {self.name: ParamSpec((self.size,), init="zeros" if self.offset else "ones")}

    def load(self, fetch):
        if self.has_weight:
            w = fetch(self.name)
            if self.offset or self.gain != 1.0:
                self.weight = ((w.float() + self.offset) * self.gain).contiguous()
            else:
                self.weight = w.contiguous()

    def rms_params(self):
        """(weight, eps) of a norm that other parts' kernels may apply themselves; a norm without a weight declines."""
        return (self.weight, self.eps) if self.has_weight else None

    def unit_params(self):
        return self.weight, self.eps

    def forward(self, h, ctx, rows=None):
        return ops.rmsnorm(h, self.weight, self.eps, ctx.act_dtype, rows=rows)


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * w + b, var the mean of the squared deviations; statistics in float32, read
    from the float32 residual stream.  It is no RMS norm: `rms_params` declines, so no part fuses it away."""
    kernel_libraries = ("elementwise",)

    def __init__(self, size: int, eps: float, name: str = "weight", bias_name: str | None = "bias"):
        """`name`, `bias_name`: what weight and bias are called behind the part's prefix; `bias_name` None: no bias."""
        self.size, self.eps = int(size), float(eps)
        self.name, self.bias_name = name, bias_name
        self.weight = self.bias = None

    def param_specs(self):
        specs = {self.name: ParamSpec((self.size,), init="ones")}
        if self.bias_name:
            specs[self.bias_name] = ParamSpec((self.size,), init="zeros")
        return specs

    def load(self, fetch):
        self.weight = fetch(self.name).float().contiguous()
        self.bias = fetch(self.bias_name).float().contiguous() if self.bias_name else None

    def forward(self, h, ctx, rows=None):
        return ops.layernorm(h, self.weight, self.bias, self.eps, ctx.act_dtype, rows=rows)

    def after_gated_add(self, h, y, gate_logits, ctx):
        """h += y * sigmoid(gate_logits), then this norm of the new rows, in one launch; None where the kernel does
        not take the rows (the caller then does the two by themselves)."""
        if self.size > ops.GATED_ADD_NORM_MAX:
            return None
        return ops.gated_add_layernorm(h, y, gate_logits, self.weight, self.bias, self.eps, ctx.act_dtype)
