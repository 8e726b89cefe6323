"""Recurrent mixers: layers that carry a fixed-size state per sequence instead of a growing cache.

The state of every live sequence sits in a slot of a pool [slots, ...] that the runner allocates and binds
(`states[run]`, one pool per pass of a looped stack); the step's Context names each sequence's slot (`state_slots`), and
a sequence whose tokens all arrive in this step starts from a zero state, whatever its slot held before.
"""
from __future__ import annotations

import math

import torch
from torch import nn

from .. import ops
from ..utils.context import get_context


class GeneralizedDeltaRule(nn.Module):
    """Per head a matrix memory S [dim, dim] in fp32, updated by every token:

        S <- diag(w) S - (a * u) (u^T S) + k v^T,      o = S^T r

    with a data-dependent decay w = exp(-decay_scale * sigmoid(w0 + W2 tanh(l))) in (0, 1) per key channel (l: a low-rank
    projection of the input), a removal rate a = sigmoid(a_raw + a_bias) along the unit key u = k / |k|, and the read-out
    normalised per head (o / rms(o) * norm) and gated by sigmoid(g).  `decay_scale` defaults to e^(-1/2).

    forward takes column views r, k, v, a_raw, g, l of the fused projection output and returns [T, H*dim] in the
    activation type, ready for the output projection (kernels: csrc/delta_rule.hip)."""

    def __init__(self, num_heads: int, head_dim: int, rank: int, eps: float, decay_scale: float = math.exp(-0.5), state_runs: int = 1):
        super().__init__()
        n = num_heads * head_dim
        self.num_heads, self.head_dim, self.rank, self.eps, self.decay_scale = num_heads, head_dim, rank, eps, decay_scale
        self.w2 = nn.Parameter(torch.zeros(n, rank), requires_grad=False)
        self.w0 = nn.Parameter(torch.zeros(n), requires_grad=False)
        self.a_bias = nn.Parameter(torch.zeros(n), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(n), requires_grad=False)
        self.state_runs = state_runs
        self.states: list = [None] * state_runs

    def state_shape(self) -> tuple[int, int, int]:
        """Shape of one sequence's state (fp32 elements); the runner allocates [slots, *state_shape()] per run."""
        return self.num_heads, self.head_dim, self.head_dim

    def forward(self, r, k, v, a_raw, g, lowrank, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        state = self.states[run]
        if state is None or ctx.state_slots is None:
            raise RuntimeError("the delta rule needs a bound state pool and a state slot per sequence")
        o = ops.delta_rule(r, k, v, a_raw, lowrank, self.w2.data, self.w0.data, self.a_bias.data, state, ctx.state_slots,
                           ctx.cu_seqlens_q, ctx.context_lens, self.num_heads, self.head_dim, self.decay_scale)
        return ops.delta_post(o, self.norm.data, g, self.num_heads, self.head_dim, self.eps)
