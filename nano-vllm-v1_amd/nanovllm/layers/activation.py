"""Gated activations over a merged [gate | up] projection: SwiGLU, silu(x[..., :I]) * x[..., I:] (reference:
nanovllm/layers/activation.py:36-58; kernel nvh_silu_mul in csrc/elementwise.hip), and its GELU counterpart with the
tanh form of GELU (kernel nvh_gelu_tanh_mul in csrc/stream_f32.hip; bf16 or fp32 rows).  ActAndMul / Act: the same for
either activation type and a choice of function (silu, gelu_tanh, relu2 = relu squared; kernel nvh_act_mul)."""
import torch
from torch import nn

from .. import ops


class SiluAndMul(nn.Module):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.silu_mul(x)


class GeluTanhAndMul(nn.Module):
    """gelu_tanh(x[..., :I]) * x[..., I:], gelu_tanh(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))), evaluated in fp32."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.gelu_tanh_mul(x)


class ActAndMul(nn.Module):
    """act(x[..., :I]) * x[..., I:] over a merged [gate | up] projection, bf16 or fp32 rows, evaluated in fp32."""

    def __init__(self, act: str = "silu"):
        super().__init__()
        assert act in ops.ACTS
        self.act = act

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.act_mul(x, self.act, True)


class Act(nn.Module):
    """An ungated activation over plain rows (relu2: max(x, 0)^2)."""

    def __init__(self, act: str = "relu2"):
        super().__init__()
        assert act in ops.ACTS
        self.act = act

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.act_mul(x, self.act, False)
