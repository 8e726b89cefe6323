"""Dinatar: a decoder-only stack of parallel layers over an fp32 residual stream, with learned absolute positions, three
kinds of sequence mixers and dense or mixture-of-experts feed-forwards, an optional looped span of layers, and a tied output
projection (the embedding table is reused for the logits).

    x_t = s_e * E[token_t] + P[t]                     (s_e: the embedding scale, P: the position table)
    for every layer run (the span [start, stop) is repeated `times` times over shared weights; caches and states are kept apart per pass):
        h = norm1(x)                                  (affine layer norm)
        x += M(h) + F(h)                              (h is computed once per layer; a layer without a feed-forward adds the mixer alone)
    logits = embed . final_norm(x) * logit_scale

Mixers (sizes and constants per layer from config.json):
  parallel  an attention branch and a recurrent branch over the one h, result = (unit(left) * left.out + unit(right) * right.out) / 2, unit = RMS over
            the width:  left = windowed softmax attention with a linear distance bias, no rotation, biased q/k/v projections
            (layers.attention.WindowedBiasAttention);  right = Mamba-2 (layers.recurrent.Mamba2)
  hgrn2     layers.recurrent.HGRN2
  gla       layers.recurrent.GatedLinearAttention, the decay logits from a low-rank pair of projections
Feed-forward: dense = down(relu(up x)^2); moe = layers.moe.SparseMoE (top-k router with bias, silu-gated experts, shared expert).

32-bit whatever the activation type: positions, the residual stream and its sums, every norm, attention scores and weights,
router logits and weights, all operands and sums of the recurrences.  Projections, convolutions and activations run in the
model's dtype (bf16, or fp32 for a model served in full precision).

config.json keys: architecture, vocab, width, max_positions, embedding.scale, logit_scale, norm.eps, loop {start, stop, times} | null,
layers[] of {type, mixer {...}, mlp {kind: dense, ff} | {kind: moe, expert {ff}, router {experts, top}, shared {ff} | null} | null}.
parallel mixer: left {heads, kv_heads, dim, vdim, scale, mask {size, keep_first}}, right {heads, vdim, state, groups, conv, norm_groups};
hgrn2: heads, dim, vdim; gla: heads, dim, vdim, tau.  Tensors: embed, pos, final.norm(.b), l<i>.norm1(.b), l<i>.mix.*, l<i>.mlp.*.
"""
from __future__ import annotations

import re
import zlib

import torch
from torch import nn

from .. import ops
from ..layers.activation import Act
from ..layers.attention import WindowedBiasAttention
from ..layers.layernorm import StreamNorm
from ..layers.linear import MergedLinear
from ..layers.moe import SparseMoE
from ..layers.recurrent import HGRN2, GatedLinearAttention, Mamba2
from .lamutar import _get, layer_runs


class DinatarAttention(nn.Module):
    def __init__(self, width: int, m, runs: int):
        super().__init__()
        h, d = int(_get(m, "heads")), int(_get(m, "dim"))
        g, dv = int(_get(m, "kv_heads", h)), int(_get(m, "vdim", d))
        mask = _get(m, "mask") or {}
        self.proj = MergedLinear(width, [h * d, g * d, g * dv], ["q", "k", "v"], bias=True)
        self.attn = WindowedBiasAttention(h, g, d, dv, float(_get(m, "scale", d ** -0.5)), WindowedBiasAttention.geometric_slopes(h),
                                          window=int(_get(mask, "size", 0) or 0), keep_first=int(_get(mask, "keep_first", 0) or 0), cache_runs=runs)
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor, run: int) -> torch.Tensor:
        return self.o(self.attn(self.proj(x), positions, run))


class DinatarMamba(nn.Module):
    def __init__(self, width: int, m, eps: float, runs: int):
        super().__init__()
        self.ssd = Mamba2(int(_get(m, "heads")), int(_get(m, "vdim")), int(_get(m, "state")), int(_get(m, "groups", 1)), int(_get(m, "conv")),
                          int(_get(m, "norm_groups", 1)), eps, state_runs=runs)
        self.proj = MergedLinear(width, [sum(self.ssd.projection_sizes())])          # one tensor in the checkpoint: z | x B C | dt
        self.o = MergedLinear(self.ssd.inner, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor, run: int) -> torch.Tensor:
        z, xbc, dt = self.proj(x).split(self.ssd.projection_sizes(), dim=-1)
        return self.o(self.ssd(z, xbc, dt, run))


class DinatarParallelMixer(nn.Module):
    """An attention branch (left) and a Mamba-2 branch (right) over one input; each output is RMS-normed over the width with its own
    weight and the mixer's result is half their sum, formed inside the layer's closing kernel (forward names its operands)."""

    def __init__(self, width: int, m, eps: float, runs: int):
        super().__init__()
        self.left = DinatarAttention(width, _get(m, "left"), runs)
        self.right = DinatarMamba(width, _get(m, "right"), eps, runs)
        self.left_out = nn.Parameter(torch.ones(width), requires_grad=False)
        self.right_out = nn.Parameter(torch.ones(width), requires_grad=False)
        self.eps = eps

    def forward(self, x: torch.Tensor, positions: torch.Tensor, run: int) -> dict:
        return dict(a=self.left(x, positions, run), a_weight=self.left_out.data, b=self.right(x, positions, run), b_weight=self.right_out.data,
                    branch_scale=0.5, branch_eps=self.eps)


class DinatarHgrn2(nn.Module):

    def __init__(self, width: int, m, eps: float, runs: int):
        super().__init__()
        h, d, dv = int(_get(m, "heads")), int(_get(m, "dim")), int(_get(m, "vdim"))
        self.proj = MergedLinear(width, [h * d, h * d, h * dv], ["q", "f", "v"])
        self.cell = HGRN2(h, d, dv, eps, state_runs=runs)
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor, run: int) -> dict:
        q, f, v = self.proj.split(self.proj(x))
        return dict(a=self.o(self.cell(q, f, v, run)))


class DinatarGla(nn.Module):

    def __init__(self, width: int, m, eps: float, runs: int, rank: int):
        super().__init__()
        h, d, dv = int(_get(m, "heads")), int(_get(m, "dim")), int(_get(m, "vdim"))
        self.proj = MergedLinear(width, [h * d, h * d, h * dv, h * dv, rank], ["q", "k", "v", "g", "a1"])
        self.cell = GatedLinearAttention(h, d, dv, rank, float(_get(m, "tau")), eps, state_runs=runs)
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor, run: int) -> dict:
        q, k, v, g, low = self.proj.split(self.proj(x))
        return dict(a=self.o(self.cell(q, k, v, g, low, run)))


class DinatarDenseMLP(nn.Module):
    """down(relu(up x)^2), ungated."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up = MergedLinear(width, [ff])
        self.act = Act("relu2")
        self.down = MergedLinear(ff, [width])

    def forward(self, x: torch.Tensor) -> dict:
        return dict(c=self.down(self.act(self.up(x))))


class DinatarMoE(nn.Module):
    def __init__(self, width: int, mlp):
        super().__init__()
        router, shared = _get(mlp, "router"), _get(mlp, "shared")
        self.moe = SparseMoE(width, int(_get(_get(mlp, "expert"), "ff")), int(_get(router, "experts")), int(_get(router, "top")),
                             shared_ff=int(_get(shared, "ff")) if shared else None, act="silu", router_bias=True)

    def forward(self, x: torch.Tensor) -> dict:
        return dict(c32=self.moe(x))


class DinatarLayer(nn.Module):
    def __init__(self, width: int, spec, eps: float, runs: int, rank: int):
        super().__init__()
        kind, mixer, mlp = _get(spec, "type"), _get(spec, "mixer"), _get(spec, "mlp")
        self.norm1 = StreamNorm(width, eps, "layer")
        if kind == "parallel":
            self.mixer = DinatarParallelMixer(width, mixer, eps, runs)
        elif kind == "hgrn2":
            self.mixer = DinatarHgrn2(width, mixer, eps, runs)
        elif kind == "gla":
            self.mixer = DinatarGla(width, mixer, eps, runs, rank)
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        self.mlp = None
        if mlp:
            mlp_kind = _get(mlp, "kind", "dense")
            if mlp_kind == "dense":
                self.mlp = DinatarDenseMLP(width, int(_get(mlp, "ff")))
            elif mlp_kind == "moe":
                self.mlp = DinatarMoE(width, mlp)
            else:
                raise ValueError(f"unknown feed-forward kind {mlp_kind!r}")


class DinatarForCausalLM(nn.Module):
    requires_cache = True            # attention reads its keys from the paged cache in every step (no packed mode)
    has_recurrent_state = True       # sequences hold a state slot; cached pages cannot stand in for a prefix
    supported_dtypes = (torch.bfloat16, torch.float32)
    DEFAULT_DECAY_RANK = 16

    def __init__(self, config) -> None:
        super().__init__()
        self.config = config
        width, vocab = int(config.width), int(config.vocab)
        eps = float(_get(config.norm, "eps", 1e-5))
        self.width, self.vocab = width, vocab
        self.embed_scale = float(_get(getattr(config, "embedding", None) or {}, "scale", 1.0))
        self.logit_scale = float(getattr(config, "logit_scale", 1.0) or 1.0)
        self.runs = layer_runs(config)
        passes = {}
        for i, t, _ in self.runs:
            passes[i] = max(passes.get(i, 0), t + 1)
        ranks = getattr(config, "decay_ranks", None) or {}
        self.embed = MergedLinear(width, [vocab])            # [vocab, width]: the table, and the output projection
        self.pos = nn.Parameter(torch.zeros(int(config.max_positions), width), requires_grad=False)
        self.layers = nn.ModuleList([DinatarLayer(width, spec, eps, passes.get(i, 1), ranks.get(i, self.DEFAULT_DECAY_RANK))
                                     for i, spec in enumerate(config.layers)])
        self.final_norm = StreamNorm(width, eps, "layer")
        self.collect = None          # a list: takes a copy of x whenever a layer run has finished (debugging, tests)

    # ------------------------------------------------------------------ checkpoint names
    def weight_target(self, name: str):
        """(parameter name, shard id | None) of a checkpoint tensor."""
        top = {"embed": "embed.weight", "pos": "pos", "final.norm": "final_norm.weight", "final.norm.b": "final_norm.bias"}
        if name in top:
            return top[name], None
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m:
            raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")
        i, rest = int(m.group(1)), m.group(2)
        p = f"layers.{i}."
        if rest in ("norm1", "norm1.b"):
            return p + ("norm1.bias" if rest.endswith(".b") else "norm1.weight"), None
        if rest.startswith("mlp."):
            return self._mlp_target(p + "mlp.", rest[4:], name)
        if not rest.startswith("mix."):
            raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")
        leaf = rest[4:]
        mixer = self.layers[i].mixer
        pm = p + "mixer."
        if isinstance(mixer, DinatarParallelMixer):
            if leaf in ("left.out", "right.out"):
                return pm + leaf.replace(".", "_"), None
            side, _, leaf = leaf.partition(".")
            if side == "left":
                if leaf == "o":
                    return pm + "left.o.weight", None
                base, _, b = leaf.partition(".")
                if base in ("q", "k", "v") and b in ("", "b"):
                    return pm + ("left.proj.bias" if b else "left.proj.weight"), base
            elif side == "right":
                direct = {"conv": "conv_weight", "conv.b": "conv_bias", "dt_bias": "dt_bias", "A_log": "A_log", "D": "D", "norm": "norm"}
                if leaf in direct:
                    return pm + "right.ssd." + direct[leaf], None
                if leaf == "o":
                    return pm + "right.o.weight", None
                if leaf == "in":
                    return pm + "right.proj.weight", None
        elif isinstance(mixer, DinatarHgrn2):
            direct = {"f.b": "cell.f_bias", "lower": "cell.lower", "norm": "cell.norm", "o": "o.weight"}
            if leaf in direct:
                return pm + direct[leaf], None
            if leaf in ("q", "f", "v"):
                return pm + "proj.weight", leaf
        elif isinstance(mixer, DinatarGla):
            direct = {"a2": "cell.decay_up.weight", "a2.b": "cell.decay_up.bias", "norm": "cell.norm", "o": "o.weight"}
            if leaf in direct:
                return pm + direct[leaf], None
            if leaf in ("q", "k", "v", "g", "a1"):
                return pm + "proj.weight", leaf
        raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")

    def _mlp_target(self, p: str, leaf: str, name: str):
        if leaf == "up":
            return p + "up.weight", None
        if leaf == "down":
            return p + "down.weight", None
        if leaf == "router":
            return p + "moe.router.weight", None
        if leaf == "router.b":
            return p + "moe.router.bias", None
        m = re.fullmatch(r"(e(\d+)|shared)\.(gate|up|down)", leaf)
        if not m:
            raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")
        if m.group(1) == "shared":
            return (p + "moe.shared.down.weight", None) if m.group(3) == "down" else (p + "moe.shared.gate_up.weight", m.group(3))
        e = int(m.group(2))
        return (p + "moe.down", e) if m.group(3) == "down" else (p + "moe.gate_up", (e, m.group(3)))

    @staticmethod
    def adapt_config(config, shapes: dict) -> None:
        """Sizes that only the checkpoint's tensor shapes give: the rank of each gla layer's low-rank decay projection
        (`shapes`: tensor name -> shape; empty without a checkpoint, then the default rank is used)."""
        ranks = {}
        for name, shape in shapes.items():
            m = re.fullmatch(r"l(\d+)\.mix\.a1", name)
            if m:
                ranks[int(m.group(1))] = int(shape[0])
        config.decay_ranks = ranks
        if not hasattr(config, "max_positions"):
            config.max_positions = int(shapes["pos"][0]) if "pos" in shapes else 4096

    @staticmethod
    def synthetic_tensors(config, seed: int = 0, std: float = 0.02, device="cuda", dtype=torch.bfloat16):
        """Random weights in checkpoint naming (for benchmarks and smoke runs without a checkpoint)."""
        width, vocab = int(config.width), int(config.vocab)
        ranks = getattr(config, "decay_ranks", None) or {}

        def mat(name, *shape, scale=std, shift=0.0):
            g = torch.Generator(device=device)
            g.manual_seed((zlib.crc32(name.encode()) ^ (seed * 0x9E3779B1)) & 0x7FFFFFFF)
            return name, (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * scale + shift).to(dtype)

        def ones(name, n):
            return name, torch.ones(n, device=device, dtype=dtype)

        def zeros(name, n):
            return name, torch.zeros(n, device=device, dtype=dtype)

        yield mat("embed", vocab, width, scale=1.0)
        yield mat("pos", int(config.max_positions), width, scale=0.1)
        yield ones("final.norm", width)
        yield zeros("final.norm.b", width)
        for i, spec in enumerate(config.layers):
            p, m, kind = f"l{i}.", _get(spec, "mixer"), _get(spec, "type")
            yield ones(p + "norm1", width)
            yield zeros(p + "norm1.b", width)
            if kind == "parallel":
                a, r = _get(m, "left"), _get(m, "right")
                h, d = int(_get(a, "heads")), int(_get(a, "dim"))
                g, dv = int(_get(a, "kv_heads", h)), int(_get(a, "vdim", d))
                for leaf, n in (("q", h * d), ("k", g * d), ("v", g * dv)):
                    yield mat(p + "mix.left." + leaf, n, width)
                    yield mat(p + "mix.left." + leaf + ".b", n, scale=0.1)
                yield mat(p + "mix.left.o", width, h * dv)
                rh, rdv, n, rg, taps = int(_get(r, "heads")), int(_get(r, "vdim")), int(_get(r, "state")), int(_get(r, "groups", 1)), int(_get(r, "conv"))
                inner, ch = rh * rdv, rh * rdv + 2 * rg * n
                yield mat(p + "mix.right.in", 2 * inner + 2 * rg * n + rh, width)
                yield mat(p + "mix.right.conv", ch, taps, scale=0.3)
                yield mat(p + "mix.right.conv.b", ch, scale=0.1)
                yield mat(p + "mix.right.dt_bias", rh, scale=0.5, shift=-2.0)
                yield mat(p + "mix.right.A_log", rh, scale=0.5)
                yield ones(p + "mix.right.D", rh)
                yield ones(p + "mix.right.norm", inner)
                yield mat(p + "mix.right.o", width, inner)
                yield ones(p + "mix.left.out", width)
                yield ones(p + "mix.right.out", width)
            elif kind == "hgrn2":
                h, d, dv = int(_get(m, "heads")), int(_get(m, "dim")), int(_get(m, "vdim"))
                yield mat(p + "mix.q", h * d, width)
                yield mat(p + "mix.f", h * d, width)
                yield mat(p + "mix.f.b", h * d, scale=1.0, shift=1.0)
                yield p + "mix.lower", torch.linspace(0.0, 0.9, h * d, device=device).to(dtype)
                yield mat(p + "mix.v", h * dv, width)
                yield ones(p + "mix.norm", dv)
                yield mat(p + "mix.o", width, h * dv)
            else:
                h, d, dv = int(_get(m, "heads")), int(_get(m, "dim")), int(_get(m, "vdim"))
                rank = ranks.get(i, DinatarForCausalLM.DEFAULT_DECAY_RANK)
                for leaf, n in (("q", h * d), ("k", h * d), ("v", h * dv), ("g", h * dv), ("a1", rank)):
                    yield mat(p + "mix." + leaf, n, width)
                yield mat(p + "mix.a2", h * d, rank, scale=0.1)
                yield mat(p + "mix.a2.b", h * d, scale=1.0, shift=3.0)
                yield ones(p + "mix.norm", dv)
                yield mat(p + "mix.o", width, h * dv)
            mlp = _get(spec, "mlp")
            if not mlp:
                continue
            if _get(mlp, "kind", "dense") == "dense":
                ff = int(_get(mlp, "ff"))
                yield mat(p + "mlp.up", ff, width)
                yield mat(p + "mlp.down", width, ff)
            else:
                ff, router, shared = int(_get(_get(mlp, "expert"), "ff")), _get(mlp, "router"), _get(mlp, "shared")
                for e in range(int(_get(router, "experts"))):
                    yield mat(f"{p}mlp.e{e}.gate", ff, width)
                    yield mat(f"{p}mlp.e{e}.up", ff, width)
                    yield mat(f"{p}mlp.e{e}.down", width, ff)
                yield mat(p + "mlp.router", int(_get(router, "experts")), width)
                yield mat(p + "mlp.router.b", int(_get(router, "experts")), scale=0.1)
                if shared:
                    sf = int(_get(shared, "ff"))
                    yield mat(p + "mlp.shared.gate", sf, width)
                    yield mat(p + "mlp.shared.up", sf, width)
                    yield mat(p + "mlp.shared.down", width, sf)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """The fp32 residual stream [T, width] after the last layer (the final norm runs on the rows that are projected)."""
        x = ops.embedding_pos_stream(input_ids, positions, self.embed.weight.data, self.pos.data, self.embed_scale)
        h = ops.residual_norm(x, **self.layers[self.runs[0][0]].norm1.spec())
        for n, (i, p, _) in enumerate(self.runs):
            layer = self.layers[i]
            terms = layer.mixer(h, positions, p)
            if layer.mlp is not None:
                terms.update(layer.mlp(h))
            nxt = self.layers[self.runs[n + 1][0]].norm1.spec() if n + 1 < len(self.runs) else {}
            h = ops.residual_norm(x, **terms, **nxt)          # the layer's close and the next layer's norm in one launch
            if self.collect is not None:
                self.collect.append(x.clone())
        return x

    def gather_rows(self, hidden: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        return ops.gather_rows_f32(hidden, rows)

    def compute_logits_rows(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits [R, vocab] of selected rows of the stream: final norm, the embedding table as the head, the logit scale."""
        h = ops.residual_norm(rows, **self.final_norm.spec())
        return ops.logits_scale(self.embed(h, out_f32=True), self.logit_scale)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.compute_logits_rows(hidden)
