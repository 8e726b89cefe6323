"""Dinatar, restated plainly: one slow function per mechanism, straight from the design's equations, in float64 on the CPU.

Nothing here is shared with the engine: no kernels, no caches, no batching.  Every function takes a whole sequence
(tokens 0..T-1 of one request) and walks it the obvious way, token by token where there is a recurrence.  `W` maps
checkpoint tensor names to tensors, `cfg` is the config.json dictionary.

Notation: D model width; per mixer H heads, G key/value heads or groups, dk query/key (or state) size, dv value size.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def _w(W, name):
    return W[name].to(F)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms_unit(x, eps):
    """x * rsqrt(mean of squares + eps) along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def embed(W, cfg, tokens):
    t = torch.as_tensor(tokens, dtype=torch.long)
    return _w(W, "embed")[t] * float(cfg["embedding"]["scale"]) + _w(W, "pos")[torch.arange(len(tokens))]


# ------------------------------------------------------------------------------------------------ mixers
def windowed_biased_attention(W, p, m, h):
    """Softmax attention without rotation: score(i, j) = scale q_i.k_j - slope_head (i - j); i sees j <= i that lie within
    the last `size` positions or among the first `keep_first` ones."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ _w(W, p + "q").T + _w(W, p + "q.b")).view(T, H, dk)
    k = (h @ _w(W, p + "k").T + _w(W, p + "k.b")).view(T, G, dk)
    v = (h @ _w(W, p + "v").T + _w(W, p + "v.b")).view(T, G, dv)
    size, keep = int(m["mask"]["size"]), int(m["mask"]["keep_first"])
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        slope = 2.0 ** (-8.0 * (head + 1) / H)
        for i in range(T):
            js = [j for j in range(i + 1) if (i - j < size or j < keep)]
            jt = torch.tensor(js)
            s = (k[jt, g] @ q[i, head]) * float(m["scale"]) - slope * (i - jt).to(F)
            a = torch.softmax(s, 0)
            out[i, head] = a @ v[jt, g]
    return out.reshape(T, H * dv) @ _w(W, p + "o").T


def mamba2(W, p, m, h, eps):
    """State-space duality layer: in-projection [z | x | B | C | dt], causal depthwise convolution + silu over x, B, C,
    per-head scalar decay exp(-exp(A_log) dt), state S [N, dv], gate silu(z) BEFORE the grouped RMS norm."""
    T = h.shape[0]
    H, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * dv
    proj = h @ _w(W, p + "in").T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    assert dt.shape[1] == H
    cw, cb = _w(W, p + "conv"), _w(W, p + "conv.b")           # [channels, taps]: last column multiplies the current token
    taps = cw.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F), xbc], 0)
    conv = torch.stack([(padded[t:t + taps].T * cw).sum(1) + cb for t in range(T)], 0)
    conv = silu(conv)
    x = conv[:, :inner].view(T, H, dv)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    C = conv[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + _w(W, p + "dt_bias"))
    A = torch.exp(_w(W, p + "A_log"))
    Dskip = _w(W, p + "D")
    y = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(N, dv, dtype=F)
        for t in range(T):
            S = torch.exp(-A[head] * dt[t, head]) * S + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S.T @ C[t, g] + Dskip[head] * x[t, head]
    y = y.reshape(T, inner) * silu(z)
    parts = int(m["norm_groups"])
    y = rms_unit(y.view(T, parts, inner // parts), eps).reshape(T, inner) * _w(W, p + "norm")
    return y @ _w(W, p + "o").T


def parallel_mixer(W, p, m, h, eps):
    left = windowed_biased_attention(W, p + "left.", m["left"], h)
    right = mamba2(W, p + "right.", m["right"], h, eps)
    return 0.5 * (rms_unit(left, eps) * _w(W, p + "left.out") + rms_unit(right, eps) * _w(W, p + "right.out"))


def hgrn2(W, p, m, h, eps):
    """HGRN2 cell: the forget gate f doubles as the write gate through its complement, S <- diag(f) S + (1 - f) v^T, o = S^T q."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ _w(W, p + "q").T).view(T, H, dk)
    v = (h @ _w(W, p + "v").T).view(T, H, dv)
    low = _w(W, p + "lower")
    f = (low + (1.0 - low) * torch.sigmoid(h @ _w(W, p + "f").T + _w(W, p + "f.b"))).view(T, H, dk)
    o = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        S = torch.zeros(dk, dv, dtype=F)
        for t in range(T):
            S = f[t, head][:, None] * S + torch.outer(1.0 - f[t, head], v[t, head])
            o[t, head] = S.T @ q[t, head]
    o = rms_unit(o, eps) * _w(W, p + "norm")
    return o.reshape(T, H * dv) @ _w(W, p + "o").T


def gla(W, p, m, h, eps):
    """Gated linear attention: per key channel a decay sigmoid(z)^(1/tau), z from a low-rank pair of projections."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ _w(W, p + "q").T).view(T, H, dk) * dk ** -0.5
    k = (h @ _w(W, p + "k").T).view(T, H, dk)
    v = (h @ _w(W, p + "v").T).view(T, H, dv)
    zz = (h @ _w(W, p + "a1").T) @ _w(W, p + "a2").T + _w(W, p + "a2.b")
    alpha = torch.exp(torch.nn.functional.logsigmoid(zz) / float(m["tau"])).view(T, H, dk)
    o = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        S = torch.zeros(dk, dv, dtype=F)
        for t in range(T):
            S = alpha[t, head][:, None] * S + torch.outer(k[t, head], v[t, head])
            o[t, head] = S.T @ q[t, head]
    o = rms_unit(o, eps) * _w(W, p + "norm")
    o = o.reshape(T, H * dv) * silu(h @ _w(W, p + "g").T)
    return o @ _w(W, p + "o").T


MIXERS = {"hgrn2": hgrn2, "gla": gla, "parallel": parallel_mixer}


# ------------------------------------------------------------------------------------------------ feed-forward
def gated_expert(W, p, h):
    return (silu(h @ _w(W, p + "gate").T) * (h @ _w(W, p + "up").T)) @ _w(W, p + "down").T


def feed_forward(W, p, mlp, h):
    if mlp["kind"] == "dense":
        return torch.relu(h @ _w(W, p + "up").T) ** 2 @ _w(W, p + "down").T
    assert mlp["kind"] == "moe"
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    logits = h @ _w(W, p + "router").T + _w(W, p + "router.b")
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        val, idx = torch.topk(logits[t], top)
        wgt = torch.softmax(val, 0)
        for e, a in zip(idx.tolist(), wgt):
            out[t] += a * gated_expert(W, f"{p}e{e}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        out = out + gated_expert(W, p + "shared.", h)
    assert E == sum(1 for n in W if n.startswith(p + "e") and n.endswith(".gate"))
    return out


def router_margin(W, p, mlp, h):
    """Smallest gap between the last chosen and the first rejected router logit over the rows of h (a test can require it to exceed the rounding of the served logits)."""
    top = int(mlp["router"]["top"])
    logits = h @ _w(W, p + "router").T + _w(W, p + "router.b")
    s = torch.sort(logits, -1, descending=True).values
    return float((s[:, top - 1] - s[:, top]).min()) if s.shape[1] > top else math.inf


# ------------------------------------------------------------------------------------------------ the stack
def layer_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def layer(W, cfg, i, x):
    """x <- x + mixer(n) + ff(n), n = norm1(x) computed once for the two sublayers."""
    spec, eps = cfg["layers"][i], float(cfg["norm"]["eps"])
    p = f"l{i}."
    n = layer_norm(x, _w(W, p + "norm1"), _w(W, p + "norm1.b"), eps)
    y = MIXERS[spec["type"]](W, p + "mix.", spec["mixer"], n, eps)
    if spec.get("mlp"):
        y = y + feed_forward(W, p + "mlp.", spec["mlp"], n)
    return x + y


def forward(W, cfg, tokens, collect=None):
    """Logits [T, vocab] of one whole sequence; `collect` (a list) takes a copy of x whenever a layer run has finished."""
    eps = float(cfg["norm"]["eps"])
    x = embed(W, cfg, tokens)
    for i in layer_order(cfg):
        x = layer(W, cfg, i, x)
        if collect is not None:
            collect.append(x.clone())
    n = layer_norm(x, _w(W, "final.norm"), _w(W, "final.norm.b"), eps)
    return n @ _w(W, "embed").T * float(cfg["logit_scale"])
