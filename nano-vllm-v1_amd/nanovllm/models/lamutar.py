"""Lamutar: a decoder-only hybrid of softmax-attention layers and generalized-delta-rule layers over an fp32 residual
stream, with a Dynamic-Tanh norm before AND after every sublayer and an optional looped span of layers.

    x = embed[token]                                  (x0 = this embedding output)
    for every layer run (layers start..stop-1 run `times` times with the same weights; each pass has its own cache/state):
        before the first layer of pass t:  x = W_in [x; x0] + step[t]
        x = x + norm1b(mixer(norm1(x)))
        x = x + norm2b(ff(norm2(x)))                  (layers without a feed-forward skip this)
    logits = cap * tanh(head(final_norm(x)) / cap)

Mixers (sizes and constants per layer from config.json):
  attention      q, k, v, gate from one merged projection; RMS norm over the whole q / k projection; partial rotary with
                 YaRN-scaled frequencies; values rotated by their position before caching and the head outputs turned
                 back; softmax(scale q.k); per-head sigmoid gate; output projection  (layers.attention.GatedValueRotaryAttention)
  general_delta  r, k, v, a, g and a low-rank decay logit from one merged projection; matrix state per head
                 (layers.recurrent.GeneralizedDeltaRule); output projection
Feed-forward: down(gelu_tanh(gate x) * up x).

What runs in 32-bit whatever the activation type: the residual stream and every norm, rotary angles, attention scores
and weights, everything inside the recurrence, the logit softcap.  Projections run in the model's dtype (bf16, or fp32
for a model served in full precision).

config.json keys: architecture, vocab, width, norm.eps, logit_softcap, loop {start, stop, times}, layers[] of
{type, mixer {...}, mlp {kind, ff} | null}; attention mixer: heads, kv_heads, dim, vdim, scale, rot {base, dims,
scaling {factor, original, fast, slow} | null}; general_delta mixer: heads, dim.  Tensors: embed, head, loop.in, loop.step,
final.norm(.b/.alpha), l<i>.norm1|norm1b|norm2|norm2b(.b/.alpha), l<i>.mix.*, l<i>.mlp.gate|up|down.
"""
from __future__ import annotations

import math
import re
import zlib

import torch
from torch import nn

from .. import ops
from ..layers.activation import GeluTanhAndMul
from ..layers.attention import GatedValueRotaryAttention
from ..layers.layernorm import DynamicTanh
from ..layers.linear import MergedLinear
from ..layers.recurrent import GeneralizedDeltaRule
from ..layers.rotary_embedding import rotary_frequencies


def _get(obj, key, default=None):
    """config.json sub-objects arrive as dicts (raw JSON) or namespaces."""
    if isinstance(obj, dict):
        return obj.get(key, default)
    return getattr(obj, key, default)


def layer_runs(config) -> list[tuple[int, int, bool]]:
    """(layer index, pass number, opens a pass?) in execution order."""
    n = len(config.layers)
    loop = getattr(config, "loop", None)
    if not loop:
        return [(i, 0, False) for i in range(n)]
    start, stop, times = int(_get(loop, "start")), int(_get(loop, "stop")), int(_get(loop, "times"))
    assert 0 <= start < stop <= n and times >= 1, f"loop {start}..{stop} x {times} does not fit {n} layers"
    runs = [(i, 0, False) for i in range(start)]
    for t in range(times):
        runs += [(i, t, i == start) for i in range(start, stop)]
    return runs + [(i, 0, False) for i in range(stop, n)]


class LamutarAttention(nn.Module):
    def __init__(self, width: int, m, eps: float, runs: int):
        super().__init__()
        h, d = int(_get(m, "heads")), int(_get(m, "dim"))
        g, dv = int(_get(m, "kv_heads", h)), int(_get(m, "vdim", d))
        rot = _get(m, "rot")
        rot_dims, base = int(_get(rot, "dims", d)), float(_get(rot, "base", 10000.0))
        qk_freq, mag = rotary_frequencies(rot_dims, base, _get(rot, "scaling"))
        value_freq, _ = rotary_frequencies(dv, base, None)
        self.proj = MergedLinear(width, [h * d, g * d, g * dv, h], ["q", "k", "v", "g"])
        self.attn = GatedValueRotaryAttention(h, g, d, dv, float(_get(m, "scale", d ** -0.5)), eps, rot_dims, qk_freq, mag, value_freq,
                                              gated=True, cache_runs=runs)
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor, run: int) -> torch.Tensor:
        return self.o(self.attn(self.proj(x), positions, run))


class LamutarDelta(nn.Module):
    def __init__(self, width: int, m, eps: float, runs: int, rank: int):
        super().__init__()
        h, d = int(_get(m, "heads")), int(_get(m, "dim"))
        n = h * d
        self.proj = MergedLinear(width, [n, n, n, n, n, rank], ["r", "k", "v", "a", "g", "w1"])
        self.rule = GeneralizedDeltaRule(h, d, rank, eps, math.exp(-0.5), state_runs=runs)
        self.o = MergedLinear(n, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor, run: int) -> torch.Tensor:
        r, k, v, a, g, low = self.proj.split(self.proj(x))
        return self.o(self.rule(r, k, v, a, g, low, run))


class LamutarMLP(nn.Module):
    def __init__(self, width: int, ff: int):
        super().__init__()
        self.gate_up = MergedLinear(width, [ff, ff], ["gate", "up"])
        self.act = GeluTanhAndMul()
        self.down = MergedLinear(ff, [width])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down(self.act(self.gate_up(x)))


class LamutarLayer(nn.Module):
    def __init__(self, width: int, spec, eps: float, runs: int, rank: int):
        super().__init__()
        kind, mixer, mlp = _get(spec, "type"), _get(spec, "mixer"), _get(spec, "mlp")
        if kind == "attention":
            self.mixer = LamutarAttention(width, mixer, eps, runs)
        elif kind == "general_delta":
            self.mixer = LamutarDelta(width, mixer, eps, runs, rank)
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        self.norm1, self.norm1b = DynamicTanh(width), DynamicTanh(width)
        self.mlp = None
        if mlp:
            assert _get(mlp, "kind", "dense") == "dense", f"feed-forward kind {_get(mlp, 'kind')!r} unsupported"
            self.mlp = LamutarMLP(width, int(_get(mlp, "ff")))
            self.norm2, self.norm2b = DynamicTanh(width), DynamicTanh(width)


class LamutarForCausalLM(nn.Module):
    requires_cache = True            # attention reads its keys from the paged cache in every step (no packed mode)
    has_recurrent_state = True       # sequences hold a state slot; cached pages cannot stand in for a prefix
    supported_dtypes = (torch.bfloat16, torch.float32)

    def __init__(self, config) -> None:
        super().__init__()
        self.config = config
        width, vocab = int(config.width), int(config.vocab)
        eps = float(_get(config.norm, "eps", 1e-6))
        self.width, self.vocab = width, vocab
        self.softcap = float(getattr(config, "logit_softcap", 0.0) or 0.0)
        self.runs = layer_runs(config)
        passes = {}
        for i, t, _ in self.runs:
            passes[i] = max(passes.get(i, 0), t + 1)
        ranks = getattr(config, "decay_ranks", None) or {}
        self.embed = MergedLinear(width, [vocab])            # [vocab, width]: a table, stored like a projection
        self.layers = nn.ModuleList([LamutarLayer(width, spec, eps, passes[i], ranks.get(i, self.DEFAULT_DECAY_RANK)) for i, spec in enumerate(config.layers)])
        self.looped = bool(getattr(config, "loop", None))
        if self.looped:
            times = int(_get(config.loop, "times"))
            self.loop_in = MergedLinear(2 * width, [width])
            self.loop_step = nn.Parameter(torch.zeros(times, width), requires_grad=False)
        self.final_norm = DynamicTanh(width)
        self.head = MergedLinear(width, [vocab])
        self.collect = None          # a list: receives a copy of the stream after every layer run (debugging, tests)

    # ------------------------------------------------------------------ checkpoint names
    _NORMS = {"": "weight", ".b": "bias", ".alpha": "alpha"}

    def weight_target(self, name: str):
        """(parameter name, shard id | None) of a checkpoint tensor."""
        top = {"embed": "embed.weight", "head": "head.weight", "loop.in": "loop_in.weight", "loop.step": "loop_step"}
        if name in top:
            return top[name], None
        m = re.fullmatch(r"final\.norm(\.b|\.alpha)?", name)
        if m:
            return "final_norm." + self._NORMS[m.group(1) or ""], None
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m:
            raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")
        i, rest = int(m.group(1)), m.group(2)
        p = f"layers.{i}."
        n = re.fullmatch(r"(norm1b|norm2b|norm1|norm2)(\.b|\.alpha)?", rest)
        if n:
            return p + n.group(1) + "." + self._NORMS[n.group(2) or ""], None
        if rest.startswith("mlp."):
            leaf = rest[4:]
            return (p + "mlp.down.weight", None) if leaf == "down" else (p + "mlp.gate_up.weight", leaf)
        assert rest.startswith("mix."), name
        leaf = rest[4:]
        attention = isinstance(self.layers[i].mixer, LamutarAttention)
        if leaf == "o":
            return p + "mixer.o.weight", None
        if attention:
            if leaf in ("q.norm", "k.norm"):
                return p + "mixer.attn." + leaf[0] + "_norm", None
            return p + "mixer.proj.weight", leaf
        direct = {"w2": "w2", "w0": "w0", "a.b": "a_bias", "norm": "norm"}
        if leaf in direct:
            return p + "mixer.rule." + direct[leaf], None
        return p + "mixer.proj.weight", leaf

    DEFAULT_DECAY_RANK = 16

    @staticmethod
    def adapt_config(config, shapes: dict) -> None:
        """Sizes that only the checkpoint's tensor shapes give: the rank of each delta layer's low-rank decay projection
        (`shapes`: tensor name -> shape; empty without a checkpoint, then the default rank is used)."""
        ranks = {}
        for name, shape in shapes.items():
            m = re.fullmatch(r"l(\d+)\.mix\.w1", name)
            if m:
                ranks[int(m.group(1))] = int(shape[0])
        config.decay_ranks = ranks

    @staticmethod
    def synthetic_tensors(config, seed: int = 0, std: float = 0.02, device="cuda", dtype=torch.bfloat16):
        """Random weights in checkpoint naming (for benchmarks and smoke runs without a checkpoint)."""
        width, vocab = int(config.width), int(config.vocab)
        ranks = getattr(config, "decay_ranks", None) or {}

        def mat(name, *shape, scale=std):
            g = torch.Generator(device=device)
            g.manual_seed((zlib.crc32(name.encode()) ^ (seed * 0x9E3779B1)) & 0x7FFFFFFF)
            return name, (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * scale).to(dtype)

        def norm(name):
            yield name, torch.ones(width, device=device, dtype=dtype)
            yield name + ".b", torch.zeros(width, device=device, dtype=dtype)
            yield name + ".alpha", torch.tensor(0.5, device=device, dtype=dtype)

        yield mat("embed", vocab, width, scale=1.0)
        yield mat("head", vocab, width)
        loop = getattr(config, "loop", None)
        if loop:
            yield mat("loop.in", width, 2 * width)
            yield mat("loop.step", int(_get(loop, "times")), width)
        yield from norm("final.norm")
        for i, spec in enumerate(config.layers):
            p, m = f"l{i}.", _get(spec, "mixer")
            for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if _get(spec, "mlp") else ()):
                yield from norm(p + nm)
            h, d = int(_get(m, "heads")), int(_get(m, "dim"))
            if _get(spec, "type") == "attention":
                g, dv = int(_get(m, "kv_heads", h)), int(_get(m, "vdim", d))
                yield mat(p + "mix.q", h * d, width)
                yield mat(p + "mix.k", g * d, width)
                yield mat(p + "mix.v", g * dv, width)
                yield mat(p + "mix.g", h, width)
                yield p + "mix.q.norm", torch.ones(h * d, device=device, dtype=dtype)
                yield p + "mix.k.norm", torch.ones(g * d, device=device, dtype=dtype)
                yield mat(p + "mix.o", width, h * dv)
            else:
                n, decay_rank = h * d, ranks.get(i, LamutarForCausalLM.DEFAULT_DECAY_RANK)
                for leaf in ("r", "k", "v", "a", "g"):
                    yield mat(p + "mix." + leaf, n, width)
                yield mat(p + "mix.w1", decay_rank, width)
                yield mat(p + "mix.w2", n, decay_rank, scale=0.1)
                yield mat(p + "mix.w0", n, scale=1.0)
                yield mat(p + "mix.a.b", n, scale=1.0)
                yield p + "mix.norm", torch.ones(n, device=device, dtype=dtype)
                yield mat(p + "mix.o", width, n)
            mlp = _get(spec, "mlp")
            if mlp:
                ff = int(_get(mlp, "ff"))
                yield mat(p + "mlp.gate", ff, width)
                yield mat(p + "mlp.up", ff, width)
                yield mat(p + "mlp.down", width, ff)

    # ------------------------------------------------------------------ forward
    def _next_norm(self, n: int):
        """The norm that opens layer run n+1, when the stream goes straight into it."""
        if n + 1 < len(self.runs) and not self.runs[n + 1][2]:
            return self.layers[self.runs[n + 1][0]].norm1.triple()
        return None

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """The fp32 residual stream [T, width] after the last layer (the final norm runs on the rows that are projected)."""
        t = input_ids.numel()
        table = self.embed.weight.data
        cat = x0 = None
        if self.looped:
            cat = torch.empty(t, 2 * self.width, dtype=table.dtype, device=table.device)     # [stream | first embedding]
            x0 = cat[:, self.width:]
        x = ops.embedding_stream(input_ids, table, x0)
        h = None
        for n, (i, p, opens) in enumerate(self.runs):
            layer = self.layers[i]
            if opens:
                ops.stream_cast_(x, cat)
                h = ops.residual_dyt(x, self.loop_in(cat), bias=self.loop_step.data[p], accumulate=False, nxt=layer.norm1.triple())
            elif h is None:
                h = ops.residual_dyt(x, nxt=layer.norm1.triple())
            y = layer.mixer(h, positions, p)
            after = layer.norm2.triple() if layer.mlp is not None else self._next_norm(n)
            h = ops.residual_dyt(x, y, post=layer.norm1b.triple(), nxt=after)
            if layer.mlp is not None:
                h = ops.residual_dyt(x, layer.mlp(h), post=layer.norm2b.triple(), nxt=self._next_norm(n))
            if self.collect is not None:
                self.collect.append(x.clone())
        return x

    def gather_rows(self, hidden: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        return ops.gather_rows_f32(hidden, rows)

    def compute_logits_rows(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits [R, vocab] of selected rows of the stream: final norm, head, softcap."""
        h = ops.residual_dyt(rows, nxt=self.final_norm.triple())
        return ops.logit_softcap(self.head(h, out_f32=True), self.softcap)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.compute_logits_rows(hidden)
