"""Norm operator modules.  RMSNorm: arithmetic in csrc/elementwise.hip (nvh_rmsnorm / nvh_add_rmsnorm).
StreamNorm: a layer norm or RMS norm of the fp32 residual stream, applied together with the residual add in front of it by
nvh_residual_norm (csrc/stream_f32.hip).
DynamicTanh: a norm without statistics, tanh(alpha x) * weight + bias, applied together with the residual add around
it by nvh_residual_dyt (csrc/stream_f32.hip) over an fp32 residual stream.

Interface of the reference's nanovllm/layers/layernorm.py:48-165: ``RMSNorm(hidden_size,
eps)``, ``.weight``, ``forward(x)`` -> y, ``forward(x, residual)`` -> (y, new_residual).
"""
import torch
from torch import nn

from .. import ops


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)

    def forward(self, x, residual: torch.Tensor | None = None):
        """x: tensor, or a SplitKOutput (unreduced projection; only with a residual)."""
        slabs = getattr(x, "slabs", None)
        if residual is None:
            if slabs is not None:
                x = x.reduce()
            return ops.rmsnorm(x, self.weight.data, self.eps)
        # the residual stream is updated in place: new_residual aliases `residual`
        if slabs is not None:
            return ops.add_rmsnorm(None, residual, self.weight.data, self.eps, partials=slabs)
        return ops.add_rmsnorm(x, residual, self.weight.data, self.eps)


class DynamicTanh(nn.Module):
    """tanh(alpha * x) * weight + bias with a learned scalar alpha; no mean, no variance, no epsilon.

    The module holds the parameters; the arithmetic runs fused with a residual add (ops.residual_dyt), which takes the
    `triple()` of the norm after the sublayer and of the norm that opens the next one."""

    def __init__(self, hidden_size: int, alpha: float = 0.5) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(hidden_size), requires_grad=False)
        self.alpha = nn.Parameter(torch.full((1,), alpha), requires_grad=False)
        self.alpha.weight_loader = lambda param, t: param.data.copy_(t.reshape(1))

    def triple(self):
        return self.alpha.data, self.weight.data, self.bias.data

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x fp32 [rows, dim] -> normalised rows in the parameters' type (x is left as it is)."""
        return ops.residual_dyt(x, nxt=self.triple())


class StreamNorm(nn.Module):
    """Norm of an fp32 residual stream with statistics: kind "layer" = (x - mean) / sqrt(var + eps) * weight + bias (var: the mean
    squared deviation), kind "rms" = x * rsqrt(mean of squares + eps) * weight.  The module holds the parameters; the arithmetic
    runs fused with the residual add that precedes it (ops.residual_norm takes `spec()`)."""

    def __init__(self, hidden_size: int, eps: float, kind: str = "layer", bias: bool = True) -> None:
        super().__init__()
        assert kind in ("layer", "rms")
        self.kind, self.eps = kind, eps
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)
        if bias and kind == "layer":
            self.bias = nn.Parameter(torch.zeros(hidden_size), requires_grad=False)
        else:
            self.register_parameter("bias", None)

    def spec(self) -> dict:
        return dict(norm=self.kind, weight=self.weight.data, bias=None if self.bias is None else self.bias.data, eps=self.eps)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x fp32 [rows, dim] -> normalised rows in the parameters' type (x is left as it is)."""
        return ops.residual_norm(x, **self.spec())
