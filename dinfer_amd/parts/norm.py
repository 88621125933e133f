"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * (w + offset), float arithmetic
(crates/layers/src/nn.rs:78-111, crates/kernels/cuda/rmsnorm_core.cuh:63-81).
LayerNorm: y = (x - mean) / sqrt(var + eps) * w + b, float arithmetic; its input (the residual stream) may be kept in
32 bits where its output is the engine's dtype."""
from __future__ import annotations

from ..kernels import ops
from .base import Norm
from .registry import NORMS
from .spec import TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, width: int, eps: float, weight_offset: float = 0.0, weight_name: str = "weight"):
        self.width, self.eps, self.weight_offset, self.weight_name = width, eps, weight_offset, weight_name
        self.weight = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.width,), init="gain")}

    def load(self, get):
        self.weight = get(self.weight_name)

    def carried(self):
        return (self.weight, self.weight_offset, self.eps)

    def forward(self, x, out, n_rows, *, residual=None, rows=None):
        if residual is None and x.dtype != out.dtype:
            # a stream kept in 32 bits, normed into the engine's dtype
            return ops.rmsnorm_stream(x, n_rows, out=out, weight=self.weight, eps=self.eps, offset=self.weight_offset,
                                      rows=rows)
        return ops.rmsnorm(x, self.weight, out, self.eps, n_rows, residual=residual, rows=rows,
                           weight_offset=self.weight_offset)


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """Tensors: weight_name and weight_name + bias_suffix (no bias tensor with bias=False)."""

    def __init__(self, width: int, eps: float, bias: bool = True, weight_name: str = "weight", bias_name: str = "bias"):
        self.width, self.eps, self.has_bias = width, eps, bias
        self.weight_name, self.bias_name = weight_name, bias_name
        self.weight = self.bias = None

    def tensors(self):
        t = {self.weight_name: TensorSpec((self.width,), init="gain")}
        if self.has_bias:
            t[self.bias_name] = TensorSpec((self.width,), init="zeros")
        return t

    def load(self, get):
        self.weight = get(self.weight_name).float()      # small parameters: kept in 32 bits (exact for bfloat16 files)
        self.bias = get(self.bias_name).float() if self.has_bias else None

    def forward(self, x, out, n_rows, *, residual=None, rows=None):
        return ops.layernorm(x, self.weight, self.bias, out, self.eps, n_rows, residual=residual, rows=rows)
