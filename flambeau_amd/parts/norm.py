"""RMSNorm.  y = x * w * rsqrt(mean(x^2) + eps), sums in 32-bit
(crates/kernels-hip/src/kernels/rmsnorm_f16.cu:40-85); the fused form that first adds the
pending delta to the residual stream follows rmsnorm_f16_add_residual.cu."""
from __future__ import annotations

from ..kernels import ops
from .base import NORMS, Norm, TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    replayable = True

    def __init__(self, hidden_size: int, eps: float, unit_offset: bool = False):
        """``unit_offset``: the weight is stored around zero and the gain is one plus it, y = x / rms(x) * (1 + w)."""
        self.hidden_size = hidden_size
        self.eps = eps
        self.unit_offset = bool(unit_offset)

    def tensors(self):
        return {"weight": TensorSpec((self.hidden_size,), "vector32", init="normal" if self.unit_offset else None)}

    def bind(self, weights, rt):
        self.rt = rt
        # (``weight`` is the gain as it multiplies: every kernel that norms, fused or not, reads this one vector)
        self.weight = (weights["weight"] + 1.0).contiguous() if self.unit_offset else weights["weight"]

    def forward(self, x, out, delta=None, store_sum=False, rows=None):
        return ops.rmsnorm(x, self.weight, out, self.eps, delta=delta, store_sum=store_sum, rows=rows)

    def after_product(self, rt, resid, product):
        """Where a kernel for the shape exists the product's kernel adds its result to the stream and
        leaves the norm in factors: x * w in the compute dtype and the sums of squares in parts.
        The product that follows multiplies by rsqrt(mean + eps) itself: no norm kernel runs."""
        return rt.gemm_add_norm(product.x, product.weight, resid, self.weight, self.eps)


@NORMS.register("dynamic_tanh")
class DynamicTanh(Norm):
    """y = tanh(alpha x) * w + b: a norm that takes no mean and no variance, so nothing crosses the values
    of a row.  ``alpha`` is one learned number, ``w`` and ``b`` vectors; ``bias=False`` leaves b out."""
    replayable = True

    def __init__(self, hidden_size: int, bias: bool = True, alpha_init: float = 0.5):
        self.hidden_size = hidden_size
        self.has_bias = bool(bias)
        self.alpha_init = float(alpha_init)

    def tensors(self):
        import torch
        a0 = self.alpha_init
        t = {"weight": TensorSpec((self.hidden_size,), "vector32"),
             "alpha": TensorSpec((), "vector32", init=lambda g, shape, device: torch.full(shape, a0, device=device) * (
                 1.0 + 0.1 * torch.randn(shape, generator=g, device=device)))}
        if self.has_bias:
            t["bias"] = TensorSpec((self.hidden_size,), "vector32", init="normal")
        return t

    def bind(self, weights, rt):
        self.rt = rt
        self.weight, self.alpha = weights["weight"], weights["alpha"].reshape(1)
        self.bias = weights.get("bias")

    def forward(self, x, out, delta=None, store_sum=False, rows=None):
        return ops.dyt(x, self.alpha, self.weight, self.bias, out, delta=delta, store_sum=store_sum, rows=rows)

    def after_product(self, rt, resid, product):
        """Where a kernel for the shape exists the product's kernel adds its result to the stream and norms the
        sum in its epilogue (nothing crosses the values of a row, so the norm is finished there): the normed
        rows come back as a tensor and no norm kernel runs."""
        return rt.gemm_add_dyt(product.x, product.weight, resid, self.alpha, self.weight, self.bias)


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * w + b over a row, var the mean of the squared deviations;
    ``bias=False`` leaves b out.  Beside ``forward`` it offers ``add_to``: the norm of a sublayer's OUTPUT
    added to the stream, for arrangements that norm what a sublayer returns and not what it reads."""
    replayable = True

    def __init__(self, hidden_size: int, eps: float, bias: bool = True):
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.has_bias = bool(bias)

    def tensors(self):
        t = {"weight": TensorSpec((self.hidden_size,), "vector32")}
        if self.has_bias:
            t["bias"] = TensorSpec((self.hidden_size,), "vector32", init="normal")
        return t

    def bind(self, weights, rt):
        self.rt = rt
        self.weight, self.bias = weights["weight"], weights.get("bias")

    def forward(self, x, out, delta=None, store_sum=False, rows=None):
        return ops.layernorm(x, self.weight, self.bias, out, self.eps, delta=delta, store_sum=store_sum, rows=rows)

    def add_to(self, resid, delta, cast=None):
        """``resid += norm(delta)``; ``cast`` (a tensor of the compute dtype, or None) receives the new stream."""
        return ops.layernorm_add(delta, self.weight, self.bias, resid, self.eps, cast=cast)
