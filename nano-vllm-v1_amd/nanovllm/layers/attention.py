"""Paged attention operator module (reference interface: nanovllm/layers/attention.py:93-249).

``Attention(num_heads, head_dim, scale, num_kv_heads)`` with ``k_cache`` / ``v_cache``
attributes that the runner binds to per-layer views [pages, 256, Hkv, D] of the KV pool, and
``forward(q, k, v) -> o`` reading the per-step Context:

  cu_seqlens_q is None        one query per sequence over the cache (graph-replay decode)
                              -> nvh_attn_decode (csrc/attention_decode.hip)
  block_tables is not None    var-len queries over the paged cache (chunked prefill, prefix
                              hits, mixed batches, eager decode) -> nvh_attn_varlen, or
                              nvh_attn_decode when every sequence has exactly one query
  block_tables is None        var-len self-attention over the packed new tokens (warm-up,
                              fresh un-chunked prefill) -> nvh_attn_varlen

New K/V rows are written to the cache first (nvh_store_kvcache) whenever a cache is bound.
"""
import torch
from torch import nn

from .. import ops
from ..utils.context import get_context


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """key/value [N, Hkv, D] (token stride free) -> cache rows slot_mapping[n]; -1 skips."""
    ops.store_kvcache(key, value, k_cache, v_cache, slot_mapping)


class Attention(nn.Module):
    def __init__(self, num_heads, head_dim, scale, num_kv_heads):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])
        self.decode_splits = 0          # 0 = heuristic per call
        self.max_context = None
        self.split_fn = None            # (batch, longest context) -> (key ranges, minimum keys per range); the runner
                                        # installs one policy for eager and graph steps

    def attend(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """Attention proper, with the new K/V already in the cache (or no cache bound)."""
        ctx = get_context()
        splits, min_range = (self.split_fn(q.shape[0], ctx.max_seqlen_k or 0) if self.split_fn is not None
                             else (self.decode_splits, 0))
        if ctx.cu_seqlens_q is None:
            return ops.attn_decode(q, self.k_cache, self.v_cache, ctx.context_lens, ctx.block_tables, self.scale,
                                   splits, self.max_context, min_range)
        if ctx.block_tables is not None:
            if ctx.max_seqlen_q == 1 and ctx.context_lens is not None:
                return ops.attn_decode(q, self.k_cache, self.v_cache, ctx.context_lens, ctx.block_tables, self.scale,
                                       splits, ctx.max_seqlen_k, min_range)
            return ops.attn_varlen(q, self.k_cache, self.v_cache, ctx.cu_seqlens_q, ctx.cu_seqlens_k,
                                   ctx.max_seqlen_q, self.scale, ctx.block_tables, ctx.max_seqlen_k or None)
        return ops.attn_varlen(q, k, v, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.max_seqlen_q, self.scale,
                               None, ctx.max_seqlen_k or None)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        if self.k_cache.numel() and self.v_cache.numel() and ctx.slot_mapping is not None and ctx.slot_mapping.numel():
            store_kvcache(k, v, self.k_cache, self.v_cache, ctx.slot_mapping)
        return self.attend(q, k, v)


class GatedValueRotaryAttention(nn.Module):
    """Paged causal attention with free head sizes (query/key `head_dim`, value `value_dim`), a partial rotary on q/k
    whose frequencies the caller supplies, optionally values that are rotated by their own position before they are
    cached (each head's output is turned back by the query's position), and optionally a per-head sigmoid output gate.

    Input is the fused projection output [T, H*dim + G*dim + G*vdim (+ H)] = q | k | v | gate; RMS norms over the WHOLE
    q and k projections run with the rotary in one launch (nvh_attn_rotary_prep), attention in a second
    (nvh_attn_paged_any).  A module that serves several passes of a looped stack owns one cache per pass:
    `k_caches[run]` [pages, page, G, dim] and `v_caches[run]` [pages, G, vdim, page] (values lie transposed within a page),
    bound by the runner (`cache_runs` of each)."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float, eps: float,
                 rot_dims: int, qk_freq: torch.Tensor, qk_mag: float, value_freq: torch.Tensor | None, gated: bool,
                 cache_runs: int = 1, interleaved: bool = False):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim = num_heads, num_kv_heads, head_dim, value_dim
        self.scale, self.eps, self.rot_dims, self.qk_mag, self.gated, self.interleaved = scale, eps, rot_dims, qk_mag, gated, interleaved
        self.q_norm = nn.Parameter(torch.ones(num_heads * head_dim), requires_grad=False)
        self.k_norm = nn.Parameter(torch.ones(num_kv_heads * head_dim), requires_grad=False)
        self.register_buffer("qk_freq", qk_freq.to(dtype=torch.float32, device=self.q_norm.device), persistent=False)
        self.register_buffer("value_freq", None if value_freq is None else value_freq.to(dtype=torch.float32, device=self.q_norm.device),
                             persistent=False)
        self.cache_runs = cache_runs
        self.k_caches: list = [None] * cache_runs
        self.v_caches: list = [None] * cache_runs

    def cache_row_elems(self) -> tuple[int, int]:
        """Elements of one token's key row and value row (what the runner sizes the page pool with)."""
        return self.num_kv_heads * self.head_dim, self.num_kv_heads * self.value_dim

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        kc, vc = self.k_caches[run], self.v_caches[run]
        if kc is None or ctx.block_tables is None:
            raise RuntimeError("this attention reads its keys from the paged cache: bind caches and give every sequence a block table")
        q, gate = ops.attn_rotary_prep(proj, self.q_norm.data, self.k_norm.data, self.eps, positions, self.qk_freq, self.qk_mag,
                                       self.rot_dims, self.value_freq, kc, vc, ctx.slot_mapping, self.num_heads, self.num_kv_heads,
                                       self.head_dim, self.value_dim, self.gated, self.interleaved, self.interleaved)
        return ops.attn_paged_any(q, kc, vc, ctx.cu_seqlens_q, ctx.context_lens, ctx.block_tables, self.scale, self.num_heads,
                                  self.num_kv_heads, self.head_dim, self.value_dim, gate, self.value_freq, self.interleaved)


class WindowedBiasAttention(nn.Module):
    """Paged causal attention without rotation whose scores carry a per-head distance bias, score = scale q.k - slope_h (i - j),
    and whose queries see a sliding window of the last `window` positions plus the first `keep_first` tokens of the sequence
    (window 0: every earlier token).  Free head sizes (query/key `head_dim`, value `value_dim`), grouped key/value heads.

    Input is the fused projection output [T, H*dim + G*dim + G*vdim] = q | k | v (biases already added).  k and v are
    scattered to their pages by nvh_attn_rotary_prep (no norm, no rotary), attention runs in nvh_attn_paged_any, which walks
    only the key tiles a query block can see.  The distance to a kept token is counted from where it really stands, so it
    grows.  Positions enter nowhere else, so the cache holds keys and values as projected.  One cache pair per pass of a
    looped stack (`cache_runs`), bound by the runner."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float, slopes, window: int = 0,
                 keep_first: int = 0, cache_runs: int = 1):
        super().__init__()
        assert num_heads % num_kv_heads == 0 and window >= 0 and keep_first >= 0
        self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim = num_heads, num_kv_heads, head_dim, value_dim
        self.scale, self.window, self.keep_first = scale, window, keep_first
        slopes = None if slopes is None else torch.as_tensor(slopes, dtype=torch.float64).to(torch.float32)
        assert slopes is None or slopes.numel() == num_heads
        self.register_buffer("slopes", None if slopes is None else slopes.to(torch.empty(0).device), persistent=False)
        self.cache_runs = cache_runs
        self.k_caches: list = [None] * cache_runs
        self.v_caches: list = [None] * cache_runs

    @staticmethod
    def geometric_slopes(num_heads: int, span: float = 8.0) -> list[float]:
        """slope_h = 2^(-span (h + 1) / H), h = 0 .. H-1: the head-wise geometric sequence of linear distance biases."""
        return [2.0 ** (-span * (h + 1) / num_heads) for h in range(num_heads)]

    def cache_row_elems(self) -> tuple[int, int]:
        return self.num_kv_heads * self.head_dim, self.num_kv_heads * self.value_dim

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        kc, vc = self.k_caches[run], self.v_caches[run]
        if kc is None or ctx.block_tables is None:
            raise RuntimeError("this attention reads its keys from the paged cache: bind caches and give every sequence a block table")
        q, _ = ops.attn_rotary_prep(proj, None, None, 0.0, positions, None, 1.0, 0, None, kc, vc, ctx.slot_mapping, self.num_heads,
                                    self.num_kv_heads, self.head_dim, self.value_dim, gated=False)
        return ops.attn_paged_any(q, kc, vc, ctx.cu_seqlens_q, ctx.context_lens, ctx.block_tables, self.scale, self.num_heads,
                                  self.num_kv_heads, self.head_dim, self.value_dim, slopes=self.slopes, window=self.window,
                                  keep_first=self.keep_first)
