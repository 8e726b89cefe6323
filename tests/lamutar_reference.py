"""Slow, plain restatement of the Lamutar design on torch-CPU in fp32: one function per mechanism, written from the
equations only and sharing nothing with the package.  Tests compare the package's GPU path against it.

Notation: T tokens of ONE sequence, positions p = 0..T-1 (or an explicit offset), width D.  Weights are a dict
name -> fp32 tensor in checkpoint naming ('l<i>.mix.q', 'l<i>.norm1.alpha', ...); linear weights are [out, in].
Every function takes and returns fp32.
"""
from __future__ import annotations

import math

import torch


def lin(w: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    return x @ w.t()


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dyt(W: dict, name: str, x: torch.Tensor) -> torch.Tensor:
    """Dynamic Tanh: tanh(alpha x) * weight + bias."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


# ----------------------------------------------------------------------------------------------- rotary
def rotary_freqs(dims: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """(frequency per pair [dims/2], magnitude factor for cos and sin) with the YaRN blend when `scaling` is given."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f.float(), 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f.float(), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor, mag: float = 1.0, interleaved: bool = False,
           sign: float = 1.0) -> torch.Tensor:
    """x [T, heads, n]: the first 2*len(freqs) dimensions of every head are turned by pos * freqs (sign -1 turns
    back); pairs are (i, i + half) or, interleaved, (2i, 2i + 1); the remaining dimensions pass."""
    half = freqs.numel()
    ang = pos.float()[:, None] * freqs[None, :] * sign                      # [T, half]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
        out[..., 0:2 * half:2] = u * c - v * s
        out[..., 1:2 * half:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:2 * half]
        out[..., :half] = u * c - v * s
        out[..., half:2 * half] = v * c + u * s
    return out


# ----------------------------------------------------------------------------------------------- mixers
def attention_mixer(W: dict, p: str, m: dict, eps: float, h: torch.Tensor, interleaved_values: bool = False) -> torch.Tensor:
    """Softmax attention of one whole sequence h [T, D] (positions 0..T-1)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    pos = torch.arange(T)
    q = rms_unit(lin(W[p + "q"], h), eps) * W[p + "q.norm"]
    k = rms_unit(lin(W[p + "k"], h), eps) * W[p + "k.norm"]
    v = lin(W[p + "v"], h)
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    rot = m["rot"]
    f, mag = rotary_freqs(rot["dims"], rot["base"], rot.get("scaling"))
    q, k = rotate(q, pos, f, mag), rotate(k, pos, f, mag)
    fv, _ = rotary_freqs(dv, rot["base"], None)
    v = rotate(v, pos, fv, 1.0, interleaved_values)
    out = torch.zeros(T, H, dv)
    causal = torch.ones(T, T, dtype=torch.bool).tril()
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].t()) * m["scale"]
        s = s.masked_fill(~causal, float("-inf"))
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    out = rotate(out, pos, fv, 1.0, interleaved_values, sign=-1.0)
    gate = torch.sigmoid(lin(W[p + "g"], h))                                # [T, H]
    out = out * gate[:, :, None]
    return lin(W[p + "o"], out.reshape(T, H * dv))


def general_delta_mixer(W: dict, p: str, m: dict, eps: float, h: torch.Tensor, state: torch.Tensor | None = None):
    """Generalized delta rule over one sequence, token by token.  Returns (output [T, D], final state [H, d, d])."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r = lin(W[p + "r"], h).view(T, H, d)
    k = lin(W[p + "k"], h).view(T, H, d)
    v = lin(W[p + "v"], h).view(T, H, d)
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(lin(W[p + "w2"], torch.tanh(lin(W[p + "w1"], h))) + W[p + "w0"])).view(T, H, d)
    a = torch.sigmoid(lin(W[p + "a"], h) + W[p + "a.b"]).view(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, d, d) if state is None else state.clone()
    o = torch.zeros(T, H, d)
    for t in range(T):
        uS = torch.einsum("hi,hij->hj", u[t], S)                             # reads the old state
        S = decay[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hij,hi->hj", S, r[t])
    o = rms_unit(o, eps).reshape(T, H * d) * W[p + "norm"]
    o = o * torch.sigmoid(lin(W[p + "g"], h))
    return lin(W[p + "o"], o), S


def dense_ff(W: dict, p: str, h: torch.Tensor) -> torch.Tensor:
    return lin(W[p + "down"], gelu_tanh(lin(W[p + "gate"], h)) * lin(W[p + "up"], h))


# ----------------------------------------------------------------------------------------------- the model
def layer_runs(cfg: dict) -> list[tuple[int, int, bool]]:
    """(layer index, pass number, first layer of a pass?) in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, 0, False) for i in range(n)]
    runs = [(i, 0, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    runs += [(i, 0, False) for i in range(loop["stop"], n)]
    return runs


def forward(cfg: dict, W: dict, tokens: list[int], collect: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; `collect` receives the residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    x0 = x.clone()
    for i, t, opens_pass in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if opens_pass:
            x = lin(W["loop.in"], torch.cat([x, x0], dim=-1)) + W["loop.step"][t]
        hin = dyt(W, p + "norm1", x)
        if L["type"] == "attention":
            y = attention_mixer(W, p + "mix.", L["mixer"], eps, hin)
        elif L["type"] == "general_delta":
            y, _ = general_delta_mixer(W, p + "mix.", L["mixer"], eps, hin)
        else:
            raise ValueError(L["type"])
        x = x + dyt(W, p + "norm1b", y)
        if L.get("mlp"):
            x = x + dyt(W, p + "norm2b", dense_ff(W, p + "mlp.", dyt(W, p + "norm2", x)))
        if collect is not None:
            collect.append(x.clone())
    logits = lin(W["head"], dyt(W, "final.norm", x))
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
