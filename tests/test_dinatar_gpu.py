"""Dinatar through the engine against the plain float64 restatement in tests/dinatar_reference.py.

Every test makes its own small configuration and random weights (written as config.json + model.safetensors into a
temporary directory, so the config reader and the loader are part of what is tested), runs a schedule through
nanovllm.trace_replay.TraceReplay (the engine's runner, page/state manager and kernels) and compares logits - and, for
single layers, the residual stream - with the reference run over each whole sequence.  fp32 serving is compared
tightly, bf16 serving within the rounding of its products.
"""
import copy
import json
import math
import os

import numpy as np
import pytest
import torch

import dinatar_reference as R

pytestmark = pytest.mark.gpu

DENSE = {"kind": "dense", "ff": 100}
MOE_A = {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 5, "top": 3}, "shared": {"ff": 40}}
MOE_B = {"kind": "moe", "expert": {"ff": 36}, "router": {"experts": 7, "top": 1}, "shared": None}
# left: grouped heads, dim != vdim, neither a multiple of 16; right: a state size no tile divides, one norm group
PAR_A = {"type": "parallel", "mlp": DENSE,
         "mixer": {"left": {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.3, "mask": {"size": 13, "keep_first": 3}},
                   "right": {"heads": 4, "vdim": 12, "state": 20, "groups": 2, "conv": 3, "norm_groups": 1}}}
# left: ungrouped heads of 16 (the matrix-core kernel in bf16), no kept tokens; right: one group, three norm groups
PAR_B = {"type": "parallel", "mlp": MOE_A,
         "mixer": {"left": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 16, "scale": 0.25, "mask": {"size": 70, "keep_first": 0}},
                   "right": {"heads": 6, "vdim": 16, "state": 16, "groups": 1, "conv": 4, "norm_groups": 3}}}
# right: channel counts and a projection row that are multiples of 8 (the convolution's 16-byte form), three taps / two taps
PAR_C = {"type": "parallel", "mlp": None,
         "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.35, "mask": {"size": 40, "keep_first": 1}},
                   "right": {"heads": 8, "vdim": 8, "state": 8, "groups": 2, "conv": 3, "norm_groups": 2}}}
PAR_D = {"type": "parallel", "mlp": DENSE,
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 24, "scale": 0.35, "mask": {"size": 9, "keep_first": 2}},
                   "right": {"heads": 16, "vdim": 4, "state": 24, "groups": 1, "conv": 2, "norm_groups": 1}}}
HGRN_A = {"type": "hgrn2", "mixer": {"heads": 3, "dim": 20, "vdim": 28}, "mlp": MOE_B}
HGRN_B = {"type": "hgrn2", "mixer": {"heads": 2, "dim": 32, "vdim": 16}, "mlp": None}
GLA_A = {"type": "gla", "mixer": {"heads": 2, "dim": 16, "vdim": 48, "tau": 8.0}, "mlp": DENSE}
GLA_B = {"type": "gla", "mixer": {"heads": 3, "dim": 12, "vdim": 20, "tau": 1.0}, "mlp": MOE_A}


def config(layers, width=96, vocab=131, loop=None, max_positions=700, embed_scale=1.7, logit_scale=0.3, eps=1e-5):
    return {"architecture": "Dinatar", "vocab": vocab, "width": width, "max_positions": max_positions, "embedding": {"scale": embed_scale},
            "logit_scale": logit_scale, "norm": {"eps": eps}, "loop": loop, "layers": copy.deepcopy(layers)}


CFG_LOOP = config([HGRN_A, PAR_A, GLA_A, PAR_B], loop={"start": 1, "stop": 3, "times": 3})
# heads of 32 / 64 (matrix-core attention in bf16), a window that spans a page border, a state size of 64
CFG_FLAT = config([{"type": "parallel", "mlp": {"kind": "dense", "ff": 256},
                    "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 64, "scale": 0.2, "mask": {"size": 300, "keep_first": 5}},
                              "right": {"heads": 4, "vdim": 32, "state": 64, "groups": 4, "conv": 2, "norm_groups": 2}}},
                   GLA_B, HGRN_B], width=128, vocab=200, embed_scale=0.8, logit_scale=1.0, eps=1e-6)


def random_weights(cfg: dict, seed: int, ranks=(8, 5)) -> dict:
    """bf16 weights in checkpoint naming; decays and gates spread so that some channels forget fast and some hardly at all."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    W = {}

    def mat(name, out, inp, scale=None):
        W[name] = torch.randn(out, inp, generator=g) * (scale if scale is not None else 1.0 / math.sqrt(inp))

    def vec(name, n, scale=1.0, shift=0.0):
        W[name] = shift + scale * torch.randn(n, generator=g)

    mat("embed", V, D, 1.0)
    mat("pos", cfg["max_positions"], D, 0.3)
    vec("final.norm", D, 0.2, 1.0)
    vec("final.norm.b", D, 0.1)
    n_gla = 0
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        vec(p + "norm1", D, 0.2, 1.0)
        vec(p + "norm1.b", D, 0.1)
        if L["type"] == "parallel":
            a, r = m["left"], m["right"]
            h, gk, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for leaf, n in (("q", h * d), ("k", gk * d), ("v", gk * dv)):
                mat(p + "mix.left." + leaf, n, D, 2.0 / math.sqrt(D))
                vec(p + "mix.left." + leaf + ".b", n, 0.3)
            mat(p + "mix.left.o", D, h * dv)
            rh, rdv, N, G, taps = r["heads"], r["vdim"], r["state"], r["groups"], r["conv"]
            inner, ch = rh * rdv, rh * rdv + 2 * G * N
            mat(p + "mix.right.in", 2 * inner + 2 * G * N + rh, D)
            mat(p + "mix.right.conv", ch, taps, 0.6)
            vec(p + "mix.right.conv.b", ch, 0.2)
            vec(p + "mix.right.dt_bias", rh, 1.0, -1.0)
            W[p + "mix.right.A_log"] = torch.linspace(-3.0, 1.0, rh)
            vec(p + "mix.right.D", rh, 0.5, 1.0)
            vec(p + "mix.right.norm", inner, 0.2, 1.0)
            mat(p + "mix.right.o", D, inner)
            vec(p + "mix.left.out", D, 0.2, 1.0)
            vec(p + "mix.right.out", D, 0.2, 1.0)
        elif L["type"] == "hgrn2":
            h, d, dv = m["heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", h * d, D)
            mat(p + "mix.f", h * d, D)
            vec(p + "mix.f.b", h * d, 1.5, 1.0)
            W[p + "mix.lower"] = torch.rand(h * d, generator=g) * 0.95
            mat(p + "mix.v", h * dv, D)
            vec(p + "mix.norm", dv, 0.2, 1.0)
            mat(p + "mix.o", D, h * dv)
        else:
            h, d, dv = m["heads"], m["dim"], m["vdim"]
            rank = ranks[n_gla % len(ranks)]
            n_gla += 1
            for leaf, n in (("q", h * d), ("k", h * d), ("v", h * dv), ("g", h * dv), ("a1", rank)):
                mat(p + "mix." + leaf, n, D)
            mat(p + "mix.a2", h * d, rank, 0.7)
            vec(p + "mix.a2.b", h * d, 2.0, 2.0)
            vec(p + "mix.norm", dv, 0.2, 1.0)
            mat(p + "mix.o", D, h * dv)
        mlp = L.get("mlp")
        if not mlp:
            continue
        if mlp["kind"] == "dense":
            mat(p + "mlp.up", mlp["ff"], D)
            mat(p + "mlp.down", D, mlp["ff"])
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            for e in range(E):
                mat(f"{p}mlp.e{e}.gate", ff, D)
                mat(f"{p}mlp.e{e}.up", ff, D)
                mat(f"{p}mlp.e{e}.down", D, ff)
            mat(p + "mlp.router", E, D, 3.0 / math.sqrt(D))          # router logits spread wide, so rounding never flips a choice
            vec(p + "mlp.router.b", E, 0.5)
            if mlp.get("shared"):
                mat(p + "mlp.shared.gate", mlp["shared"]["ff"], D)
                mat(p + "mlp.shared.up", mlp["shared"]["ff"], D)
                mat(p + "mlp.shared.down", D, mlp["shared"]["ff"])
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def write_model(path, cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


class Case:
    """A model on disk, its reference weights and cached reference logits per token list."""

    def __init__(self, tmp, cfg, seed=0, weights=None):
        self.cfg = cfg
        w = weights if weights is not None else random_weights(cfg, seed)
        self.path = write_model(tmp, cfg, w)
        self.W = {k: v.double() for k, v in w.items()}
        self._ref = {}

    def ref(self, tokens):
        key = tuple(tokens)
        if key not in self._ref:
            self._ref[key] = R.forward(self.W, self.cfg, list(tokens)).numpy()
        return self._ref[key]

    def replay(self, dtype="float32", max_tokens=2048, slots=4):
        from nanovllm.trace_replay import TraceReplay
        return TraceReplay(self.path, dtype, max_tokens, slots)


def tokens_of(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def rel_err(got, want):
    """Largest row error, mean removed, relative to the spread of the reference logits."""
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / want.std())


TOL = {"float32": 2e-4, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def loop_case(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("dinatar_loop"), CFG_LOOP, seed=1)


@pytest.fixture(scope="module")
def flat_case(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("dinatar_flat"), CFG_FLAT, seed=2)


def run_schedule(rp, case, requests: dict, schedule: list, dtype: str, tol=None):
    """schedule: list of steps, each a list of (request id, token count); every position's logits are asked for and
    compared with the reference of the whole request.  Requests end when their tokens are used up."""
    at = {r: 0 for r in requests}
    worst = 0.0
    for step in schedule:
        entries, spans, end = [], [], []
        for rid, count in step:
            lo, hi = at[rid], at[rid] + count
            entries.append({"id": rid, "tokens": requests[rid][lo:hi], "want": list(range(count))})
            spans.append((rid, lo, hi))
            at[rid] = hi
            if hi == len(requests[rid]):
                end.append(rid)
        got = rp.step(entries, end)
        row = 0
        for rid, lo, hi in spans:
            want = case.ref(requests[rid])[lo:hi]
            err = rel_err(got[row:row + hi - lo], want)
            assert err < (tol or TOL[dtype]), f"request {rid} tokens {lo}..{hi}: error {err:.3g}"
            worst = max(worst, err)
            row += hi - lo
    assert all(at[r] == len(requests[r]) for r in requests)
    return worst


# ----------------------------------------------------------------------------------------------------- single mechanisms
@pytest.mark.parametrize("layer", [PAR_A, PAR_B, PAR_C, PAR_D, HGRN_A, HGRN_B, GLA_A, GLA_B],
                         ids=["parallel(gqa, ragged sizes)+dense", "parallel(heads of 16)+moe", "parallel(3 taps, aligned)", "parallel(2 taps, aligned)+dense",
                              "hgrn2+moe(top 1)", "hgrn2", "gla+dense", "gla+moe"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_stream_matches(tmp_path, layer, dtype):
    """One layer of each kind, no loop: the residual stream after it and the logits."""
    cfg = config([layer], width=72, vocab=50, embed_scale=0.6, logit_scale=2.0)
    case = Case(tmp_path, cfg, seed=3)
    toks = tokens_of(cfg, 70, 5)
    rp = case.replay(dtype)
    try:
        rp.runner.model.collect = []
        got = rp.step([{"id": 0, "tokens": toks, "want": list(range(len(toks)))}], [0])
        stream = rp.runner.model.collect[0].cpu().numpy()
    finally:
        rp.close()
    col = []
    want = R.forward(case.W, cfg, toks, col).numpy()
    assert np.abs(stream - col[0].numpy()).max() < (1e-4 if dtype == "float32" else 0.15) * max(1.0, float(col[0].abs().max()))
    assert rel_err(got, want) < TOL[dtype]


def test_loop_passes_keep_separate_caches_and_states(loop_case):
    """A looped span (three passes over a parallel and a gla layer): every layer run against the reference."""
    toks = tokens_of(CFG_LOOP, 40, 7)
    rp = loop_case.replay("float32")
    try:
        rp.runner.model.collect = []
        rp.step([{"id": 0, "tokens": toks, "want": [0]}], [0])
        streams = [c.cpu().numpy() for c in rp.runner.model.collect]
    finally:
        rp.close()
    col = []
    R.forward(loop_case.W, CFG_LOOP, toks, col)
    assert len(streams) == len(col) == 1 + 2 * 3 + 1
    for n, (a, b) in enumerate(zip(streams, col)):
        assert np.abs(a - b.numpy()).max() < 2e-4 * max(1.0, float(b.abs().max())), f"layer run {n}"


def test_scan_against_the_recurrence_written_out():
    """The diagonal-decay scan alone: grouped q/k, a decay per channel or per head, write strength, skip weight; key sizes that
    are and are not multiples of 16 and of 4; two sequences, one continued from a state, one fresh, in slots out of order."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(0)
    for H, G, dk, dv, scalar, lens in [(4, 2, 20, 12, True, [9, 5]), (2, 2, 16, 48, False, [9, 5]), (3, 1, 64, 70, True, [9, 5]), (2, 2, 37, 5, False, [9, 5]),
                                       (1, 1, 128, 64, False, [9, 5]), (1, 1, 300, 6, False, [9, 5]), (1, 1, 512, 20, True, [9, 5]),
                                       # long portions: walked in segments that are joined afterwards (beside a short one that is not)
                                       (2, 1, 32, 24, True, [300, 7]), (1, 1, 64, 16, False, [1, 555]), (2, 2, 16, 8, False, [256, 257])]:
        past = [4, 0]
        T = sum(lens)
        q, k = torch.randn(T, G * dk, generator=g), torch.randn(T, G * dk, generator=g)
        w = torch.rand(T, H if scalar else H * dk, generator=g) ** (0.02 if max(lens) > 100 else 1.0)     # (long runs: decays near one, so far tokens count)
        c = torch.rand(T, H, generator=g) + 0.5
        v = torch.randn(T, H * dv, generator=g)
        d = torch.randn(H, generator=g)
        state = torch.randn(5, H, dk, dv, generator=g)
        slots = [3, 1]
        want, new_state = torch.zeros(T, H * dv, dtype=torch.float64), state.double().clone()
        t0 = 0
        for b, n in enumerate(lens):
            for h in range(H):
                S = state[slots[b], h].double() if past[b] else torch.zeros(dk, dv, dtype=torch.float64)
                gq = h // (H // G)
                for t in range(t0, t0 + n):
                    wt = (w[t, h] if scalar else w[t, h * dk:(h + 1) * dk]).double()
                    S = (wt * S.T).T + torch.outer(c[t, h].double() * k[t, gq * dk:(gq + 1) * dk].double(), v[t, h * dv:(h + 1) * dv].double())
                    want[t, h * dv:(h + 1) * dv] = S.T @ q[t, gq * dk:(gq + 1) * dk].double() + d[h].double() * v[t, h * dv:(h + 1) * dv].double()
                new_state[slots[b], h] = S
            t0 += n
        st = state.transpose(2, 3).contiguous().cuda()          # the pool holds S transposed: [slots, H, dv, dk]
        cu = torch.tensor([0, lens[0], T], dtype=torch.int32).cuda()
        ctx = torch.tensor([lens[0] + past[0], lens[1] + past[1]], dtype=torch.int32).cuda()
        got = ops.gated_linear_scan(q.cuda(), k.cuda(), w.cuda(), v.cuda(), st, torch.tensor(slots, dtype=torch.int32).cuda(), cu, ctx, H, dk, dv, G,
                                    kscale=c.cuda(), skip=d.cuda(), max_seqlen_q=max(lens))
        assert (got.cpu().double() - want).abs().max() < 1e-4 * max(1.0, float(want.abs().max())), (H, G, dk, dv)
        assert (st.cpu().double().transpose(2, 3) - new_state).abs().max() < 1e-4 * max(1.0, float(new_state.abs().max()))


def test_router_picks_the_largest_and_weighs_them_alone():
    from nanovllm import ops
    g = torch.Generator().manual_seed(1)
    for E, top in [(5, 3), (7, 1), (64, 2), (130, 8), (3, 3)]:
        z = torch.randn(33, E, generator=g)
        ids, wts = ops.moe_route(z.cuda(), top)
        val, idx = torch.topk(z, top, dim=-1)
        assert torch.equal(ids.cpu().long(), idx)
        assert (wts.cpu() - torch.softmax(val, -1)).abs().max() < 1e-6
        # the router's product inside the same launch, both activation types
        x, w, b = torch.randn(33, 70, generator=g), torch.randn(E, 70, generator=g), torch.randn(E, generator=g)
        for cast in (torch.float32, torch.bfloat16):
            xa, wa, ba = x.to(cast), w.to(cast), b.to(cast)
            zz = xa.double() @ wa.double().T + ba.double()
            ids, wts, lg = ops.moe_route_linear(xa.cuda(), wa.cuda(), ba.cuda(), top, want_logits=True)
            assert (lg.cpu().double() - zz).abs().max() < 1e-4
            val, idx = torch.topk(lg.cpu(), top, dim=-1)
            assert torch.equal(ids.cpu().long(), idx) and (wts.cpu() - torch.softmax(val, -1)).abs().max() < 1e-6
    z = torch.tensor([[1.0, 3.0, 3.0, 0.0]])
    ids, _ = ops.moe_route(z.cuda(), 2)
    assert ids.cpu().tolist() == [[1, 2]]                     # a tie: the lower expert first


def test_grouped_product_matches_one_product_per_expert():
    """Tokens spread unevenly over experts (one expert with more than a tile, one with none): both types, ragged sizes."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(2)
    T, E, top, K, N = 150, 6, 2, 40, 52
    x, w = torch.randn(T, K, generator=g), torch.randn(E, N, K, generator=g)
    ids = torch.randint(0, 3, (T, top), generator=g).int()
    ids[:, 1] = torch.where(torch.arange(T) % 10 == 0, 5, 0).int()        # expert 0 takes most second choices, expert 4 nothing
    wts = torch.rand(T, top, generator=g)
    for cast, tol in ((torch.float32, 1e-4), (torch.bfloat16, 3e-2)):
        xa, wa = x.to(cast), w.to(cast)
        plan = ops.moe_align(ids.cuda(), E)
        y = ops.linear_grouped(xa.cuda(), wa.cuda(), plan, gather=True)
        out = ops.moe_combine(y, plan, wts.cuda()).cpu()
        want = torch.zeros(T, N)
        for t in range(T):
            for r in range(top):
                want[t] += wts[t, r] * (xa[t].float() @ wa[ids[t, r]].float().T)
        assert (out - want).abs().max() < tol * max(1.0, float(want.abs().max()))
        pos = plan["pos_of_pair"].cpu().view(T, top)
        assert sorted(pos.flatten().tolist()) == list(range(T * top))
        assert torch.equal(plan["src_token"].cpu()[pos.flatten().long()], torch.arange(T).repeat_interleave(top).int())


def test_layer_close_kernel_against_its_formula():
    from nanovllm import ops
    g = torch.Generator().manual_seed(3)
    for dim in (50, 96, 1000):
        x, a, b, c = (torch.randn(9, dim, generator=g) for _ in range(4))
        c32 = torch.randn(9, dim, generator=g)
        wa, wb, nw, nb = (torch.randn(dim, generator=g) for _ in range(4))
        unit = lambda v: v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-5)
        s = x + (0.5 * (unit(a) * wa + unit(b) * wb) + c + c32)
        mu = s.mean(-1, keepdim=True)
        want = (s - mu) / torch.sqrt(((s - mu) ** 2).mean(-1, keepdim=True) + 1e-5) * nw + nb
        xg = x.cuda()
        h = ops.residual_norm(xg, a=a.cuda(), a_weight=wa.cuda(), b=b.cuda(), b_weight=wb.cuda(), branch_scale=0.5, branch_eps=1e-5, c=c.cuda(),
                              c32=c32.cuda(), norm="layer", weight=nw.cuda(), bias=nb.cuda(), eps=1e-5)
        assert (xg.cpu() - s).abs().max() < 1e-5 and (h.cpu() - want).abs().max() < 1e-4
        xg = x.cuda()
        h = ops.residual_norm(xg, a=a.cuda(), norm="rms", weight=nw.cuda(), eps=1e-6)
        assert (h.cpu() - unit(x + a) * nw).abs().max() < 1e-4 and (xg.cpu() - (x + a)).abs().max() < 1e-6


def test_grouped_norm_with_gates_before_and_after():
    """Groups small (a wave each) and large (a workgroup each), a weight per group or per column, silu gate first, sigmoid gate last."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(4)
    unit = lambda v: v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-5)
    for groups, gs in [(3, 20), (2, 64), (1, 600), (2, 2048), (1, 2500)]:
        o, gate = torch.randn(7, groups * gs, generator=g), torch.randn(7, 2 * groups * gs, generator=g)[:, groups * gs:]
        for w in (torch.randn(gs, generator=g), torch.randn(groups * gs, generator=g)):
            wf = (w if w.numel() == groups * gs else w.repeat(groups))
            first = (unit((o * torch.nn.functional.silu(gate)).view(7, groups, gs)).reshape(7, -1) * wf)
            last = unit(o.view(7, groups, gs)).reshape(7, -1) * wf * torch.sigmoid(gate)
            plain = unit(o.view(7, groups, gs)).reshape(7, -1) * wf
            gc = gate.cuda()
            assert (ops.group_rmsnorm_gate(o.cuda(), w.cuda(), gs, 1e-5, gc, "silu", gate_first=True).cpu() - first).abs().max() < 1e-4
            assert (ops.group_rmsnorm_gate(o.cuda(), w.cuda(), gs, 1e-5, gc, "sigmoid", gate_first=False).cpu() - last).abs().max() < 1e-4
            assert (ops.group_rmsnorm_gate(o.cuda(), w.cuda(), gs, 1e-5).cpu() - plain).abs().max() < 1e-4


# ----------------------------------------------------------------------------------------------------- schedules
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_then_token_by_token(loop_case, dtype):
    toks = tokens_of(CFG_LOOP, 90, 11)
    rp = loop_case.replay(dtype)
    try:
        run_schedule(rp, loop_case, {"a": toks}, [[("a", 50)]] + [[("a", 1)]] * 40, dtype)
        # the first tokens of a sequence, one by one from the very start (shorter than the convolution, the kept tokens, the window)
        run_schedule(rp, loop_case, {"b": toks[:20]}, [[("b", 1)]] * 20, dtype)
    finally:
        rp.close()


def test_portions_of_every_size_give_the_same_logits(loop_case):
    toks = tokens_of(CFG_LOOP, 120, 13)
    rp = loop_case.replay("float32")
    try:
        for sizes in ([120], [2] * 60, [3, 2, 17, 2, 33, 16, 2, 45], [64, 56], [1, 119]):
            assert sum(sizes) == 120
            run_schedule(rp, loop_case, {"a": toks}, [[("a", s)] for s in sizes], "float32")
    finally:
        rp.close()


def test_cutting_does_not_change_a_bit_of_the_recurrent_path(tmp_path):
    """Recurrent mixers only (no attention, whose key tiles see the cut): one piece, portions and single tokens give
    identical logits, the convolution's carried inputs included."""
    cfg = config([HGRN_B, GLA_A, copy.deepcopy(PAR_A), copy.deepcopy(PAR_C)], width=64, vocab=64)
    w = random_weights(cfg, 5)
    w["l2.mix.left.out"] = torch.zeros_like(w["l2.mix.left.out"])            # the attention branches are switched off
    w["l3.mix.left.out"] = torch.zeros_like(w["l3.mix.left.out"])
    case = Case(tmp_path, cfg, weights=w)
    toks = tokens_of(cfg, 48, 2)
    rp = case.replay("float32")
    try:
        whole = rp.step([{"id": 0, "tokens": toks, "want": [47]}], [0])
        rp.step([{"id": 1, "tokens": toks[:20], "want": []}])
        rp.step([{"id": 1, "tokens": toks[20:41], "want": []}])
        for p in range(41, 47):
            rp.step([{"id": 1, "tokens": toks[p:p + 1], "want": []}])
        cut = rp.step([{"id": 1, "tokens": toks[47:], "want": [0]}], [1])
    finally:
        rp.close()
    assert np.array_equal(whole, cut)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_of_unequal_requests(loop_case, dtype):
    reqs = {"a": tokens_of(CFG_LOOP, 75, 21), "b": tokens_of(CFG_LOOP, 9, 22), "c": tokens_of(CFG_LOOP, 33, 23), "d": tokens_of(CFG_LOOP, 2, 24)}
    sched = [[("a", 30), ("b", 3)], [("a", 1), ("b", 2), ("c", 20)], [("b", 1), ("a", 17), ("c", 1), ("d", 2)], [("c", 2), ("a", 27), ("b", 3)],
             [("c", 10)]]
    rp = loop_case.replay(dtype)
    try:
        run_schedule(rp, loop_case, reqs, sched, dtype)
    finally:
        rp.close()


def test_pages_and_slots_are_used_again(flat_case):
    """A pool of three pages and two state slots serves six requests one after another and in pairs: every request after
    the first two runs on pages and slots (recurrent states, convolution inputs) that others have left behind."""
    reqs = {i: tokens_of(CFG_FLAT, n, 30 + i) for i, n in enumerate([300, 120, 257, 40, 256, 130])}
    rp = flat_case.replay("float32", max_tokens=256, slots=2)            # ceil(256/256) + 2 = 3 pages
    assert len(rp.scheduler.block_manager.blocks) == 3 and rp.scheduler.block_manager.num_state_slots == 2
    try:
        run_schedule(rp, flat_case, {0: reqs[0]}, [[(0, 200)], [(0, 100)]], "float32")
        run_schedule(rp, flat_case, {1: reqs[1], 2: reqs[2]}, [[(1, 100), (2, 7)], [(1, 20), (2, 250)]], "float32")
        run_schedule(rp, flat_case, {3: reqs[3], 4: reqs[4]}, [[(4, 255), (3, 39)], [(3, 1), (4, 1)]], "float32")
        run_schedule(rp, flat_case, {5: reqs[5]}, [[(5, 129)], [(5, 1)]], "float32")
        assert len(rp.scheduler.block_manager.free_block_ids) == 3 and len(rp.scheduler.block_manager.free_state_slots) == 2
    finally:
        rp.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_page_borders_in_prompts_and_in_decoding(flat_case, dtype):
    """Portions that end one token before, at and after a page border; decoding across it with the window (300) reaching back
    over the border; a second page border, where the window's start lies in the first page's middle."""
    toks = tokens_of(CFG_FLAT, 530, 41)
    rp = flat_case.replay(dtype, max_tokens=1100)
    try:
        run_schedule(rp, flat_case, {"a": toks}, [[("a", 255)], [("a", 1)], [("a", 1)], [("a", 2)], [("a", 251)], [("a", 3)]] + [[("a", 1)]] * 17, dtype)
        run_schedule(rp, flat_case, {"b": toks[:300]}, [[("b", 256)], [("b", 44)]], dtype)
    finally:
        rp.close()


def test_long_decoding(loop_case):
    """Far more decoded tokens than either window (13, 70): only decoded tokens are left inside the windows by the end."""
    toks = tokens_of(CFG_LOOP, 230, 43)
    rp = loop_case.replay("float32", max_tokens=512)
    try:
        run_schedule(rp, loop_case, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 225, "float32")
    finally:
        rp.close()


# ----------------------------------------------------------------------------------------------------- faults that random weights would hide
def sharp_window_case(tmp, size, keep, heads=2, dim=32):
    """One parallel layer whose recurrent branch is switched off (right.out = 0) and whose keys equal its queries (same
    weights and biases) under a large scale: a query puts nearly all its weight on the earlier occurrence of its own token -
    if the mask lets it see that token."""
    layer = {"type": "parallel", "mlp": None,
             "mixer": {"left": {"heads": heads, "kv_heads": heads, "dim": dim, "vdim": dim, "scale": 1.5, "mask": {"size": size, "keep_first": keep}},
                       "right": {"heads": 2, "vdim": 8, "state": 8, "groups": 1, "conv": 2, "norm_groups": 1}}}
    cfg = config([layer], width=64, vocab=900, max_positions=800, embed_scale=1.0, logit_scale=1.0)
    w = random_weights(cfg, 9)
    w["l0.mix.left.k"] = w["l0.mix.left.q"].clone()
    w["l0.mix.left.k.b"] = w["l0.mix.left.q.b"].clone()
    w["l0.mix.left.v"] = w["l0.mix.left.v"] * 4
    w["l0.mix.right.out"] = torch.zeros_like(w["l0.mix.right.out"])
    w["pos"] = w["pos"] * 0.05                               # positions hardly move the queries: equal tokens stay alike
    return Case(tmp, cfg, weights=w), cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_just_inside_and_just_outside_the_window_and_the_kept_tokens(tmp_path, dtype):
    """The last token repeats an earlier one.  Where the mask shows that one (the window's last position, a page border inside
    the window, the last kept token) the logits differ clearly from those of a prompt without the repeat; one position
    further (just outside the window, the first token after the kept ones) they must equal the reference that cannot see it.
    Checked for the whole prompt in one step and for the last token decoded alone."""
    size, keep, n = 260, 6, 600
    case, cfg = sharp_window_case(tmp_path, size, keep)
    base = list(range(1, n + 1))
    last = n - 1
    seen = [last - 1, last - size + 1, 512, 511, last - 255, keep - 1, 0]
    unseen = [last - size, last - size - 1, keep, 256, 255]
    rp = case.replay(dtype, max_tokens=1300)
    try:
        for far in seen + unseen:
            toks = base[:last] + [base[far]]
            ref = case.ref(toks)[-1:]
            blind = case.ref(base[:last] + [899])[-1:]
            if far in seen:
                assert rel_err(blind, ref) > 0.3, far       # the key matters: without it the logits are others
            whole = rp.step([{"id": 0, "tokens": toks, "want": [last]}], [0])
            rp.step([{"id": 1, "tokens": toks[:last], "want": []}])
            decoded = rp.step([{"id": 1, "tokens": toks[last:], "want": [0]}], [1])
            tol = TOL[dtype] if dtype == "float32" else 0.15      # (sharp weights magnify the rounding of bf16 scores)
            assert rel_err(whole, ref) < tol and rel_err(decoded, ref) < tol, far
    finally:
        rp.close()


def test_window_edges_inside_prompt_portions(tmp_path):
    """The same with small windows so that the edge falls inside 64-key tiles and between query blocks: every position of a
    prompt of repeated tokens, cut into portions, for windows of 1, 2, 63, 64, 65 with 0, 1 and 70 kept tokens."""
    for size, keep in [(1, 0), (2, 1), (63, 0), (64, 70), (65, 1)]:
        case, cfg = sharp_window_case(tmp_path / f"w{size}_{keep}", size, keep, heads=1, dim=16)
        toks = [1 + (i * 7) % 23 for i in range(200)]           # every token comes back every 23 positions
        for dtype in ("float32", "bfloat16"):
            rp = case.replay(dtype, max_tokens=512)
            try:
                run_schedule(rp, case, {"a": toks}, [[("a", 130)], [("a", 2)], [("a", 67)], [("a", 1)]], dtype, tol=None if dtype == "float32" else 0.15)
            finally:
                rp.close()


def test_distance_bias_uses_true_positions_of_kept_tokens(tmp_path):
    """Queries and keys all equal (zero weights, a bias only): the scores are the distance bias alone, so the weights of the
    kept first tokens against those of the window depend on their true distance."""
    size, keep = 10, 4
    case, cfg = sharp_window_case(tmp_path, size, keep)
    w = {k: v.to(torch.bfloat16) for k, v in case.W.items()}
    w["l0.mix.left.q"] = torch.zeros_like(w["l0.mix.left.q"])
    w["l0.mix.left.k"] = torch.zeros_like(w["l0.mix.left.k"])
    case = Case(tmp_path / "flat_scores", cfg, weights=w)
    toks = tokens_of(cfg, 90, 3)
    rp = case.replay("float32", max_tokens=256)
    try:
        run_schedule(rp, case, {"a": toks}, [[("a", 40)], [("a", 30)]] + [[("a", 1)]] * 20, "float32")
    finally:
        rp.close()


def test_recurrent_states_carry_a_token_from_far_back(tmp_path):
    """Gates near one keep a channel's memory for hundreds of tokens: the first token still shapes the last logits in each of
    the three recurrent mixers, and a state that were lost or reset between portions would show."""
    par = copy.deepcopy(PAR_B)
    par["mlp"] = None
    for kind, layer in (("hgrn2", HGRN_B), ("gla", {"type": "gla", "mixer": {"heads": 2, "dim": 16, "vdim": 16, "tau": 16.0}, "mlp": None}), ("mamba", par)):
        cfg = config([layer], width=48, vocab=90, max_positions=512, embed_scale=1.0, logit_scale=1.0)
        w = random_weights(cfg, 4)
        if kind == "hgrn2":
            w["l0.mix.lower"] = torch.full_like(w["l0.mix.lower"], 0.996)
        elif kind == "gla":
            w["l0.mix.a2.b"] = torch.full_like(w["l0.mix.a2.b"], 4.0)
            w["l0.mix.a2"] = w["l0.mix.a2"] * 0.1
        else:
            w["l0.mix.left.out"] = torch.zeros_like(w["l0.mix.left.out"])
            w["l0.mix.right.A_log"] = torch.full_like(w["l0.mix.right.A_log"], -5.0)
            w["l0.mix.right.dt_bias"] = torch.full_like(w["l0.mix.right.dt_bias"], -1.0)
        case = Case(tmp_path / kind, cfg, weights=w)
        toks = tokens_of(cfg, 400, 8)
        changed = [(toks[0] + 1) % 90] + toks[1:]
        assert rel_err(case.ref(changed)[-1:], case.ref(toks)[-1:]) > 5 * TOL["float32"], kind      # 400 tokens later it still shows
        rp = case.replay("float32", max_tokens=1024)
        try:
            run_schedule(rp, case, {"a": toks}, [[("a", 100)], [("a", 156)], [("a", 1)], [("a", 140)], [("a", 2)], [("a", 1)]], "float32")
            # portions long enough to be scanned in segments, beside a short request; then the state they left is decoded from
            run_schedule(rp, case, {"b": toks, "c": toks[:9]}, [[("b", 290), ("c", 8)], [("b", 109), ("c", 1)], [("b", 1)]], "float32")
        finally:
            rp.close()


def test_a_far_key_inside_a_wide_window(tmp_path):
    """A window wider than the prompt: the one earlier occurrence among hundreds of keys decides the output, wherever it lies."""
    case, cfg = sharp_window_case(tmp_path, 2000, 0)
    n = 600
    base = list(range(1, n + 1))
    rp = case.replay("bfloat16", max_tokens=1300)
    try:
        for far in (0, 3, 255, 256, 257, 511, 512):
            toks = base[:n - 1] + [base[far]]
            ref = case.ref(toks)[-1:]
            assert rel_err(case.ref(base[:n - 1] + [899])[-1:], ref) > 0.3
            whole = rp.step([{"id": 0, "tokens": toks, "want": [n - 1]}], [0])
            rp.step([{"id": 1, "tokens": toks[:n - 1], "want": []}])
            decoded = rp.step([{"id": 1, "tokens": toks[n - 1:], "want": [0]}], [1])
            assert rel_err(whole, ref) < 0.15 and rel_err(decoded, ref) < 0.15, far
    finally:
        rp.close()


# ----------------------------------------------------------------------------------------------------- other sizes
def test_sizes_no_kernel_tile_divides(tmp_path):
    """A width that is no multiple of 8, one key/value head, value heads of 256, one expert of which one is taken, a
    convolution of one tap and of six, eight norm groups, a loop of one pass over everything, scales of one."""
    layers = [{"type": "parallel", "mlp": {"kind": "moe", "expert": {"ff": 10}, "router": {"experts": 1, "top": 1}, "shared": {"ff": 6}},
               "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 10, "vdim": 256, "scale": 0.5, "mask": {"size": 1000, "keep_first": 1000}},
                         "right": {"heads": 8, "vdim": 6, "state": 5, "groups": 8, "conv": 1, "norm_groups": 8}}},
              {"type": "hgrn2", "mixer": {"heads": 1, "dim": 130, "vdim": 3}, "mlp": {"kind": "dense", "ff": 34}},
              {"type": "parallel", "mlp": None,
               "mixer": {"left": {"heads": 3, "kv_heads": 3, "dim": 256, "vdim": 16, "scale": 0.05, "mask": {"size": 5, "keep_first": 2}},
                         "right": {"heads": 1, "vdim": 64, "state": 128, "groups": 1, "conv": 6, "norm_groups": 1}}},
              {"type": "gla", "mixer": {"heads": 1, "dim": 48, "vdim": 10, "tau": 2.5}, "mlp": None}]
    cfg = config(layers, width=50, vocab=37, loop={"start": 0, "stop": 4, "times": 1}, max_positions=100, embed_scale=1.0, logit_scale=1.0)
    case = Case(tmp_path, cfg, weights=random_weights(cfg, 6, ranks=(3,)))
    toks = tokens_of(cfg, 80, 3)
    for dtype in ("float32", "bfloat16"):
        rp = case.replay(dtype)
        try:
            run_schedule(rp, case, {"a": toks, "b": toks[:7]}, [[("a", 33), ("b", 5)], [("a", 1), ("b", 2)], [("a", 46)]], dtype)
        finally:
            rp.close()


def test_config_without_a_loop_entry(tmp_path):
    cfg = config([GLA_A, HGRN_A], width=64, vocab=40)
    del cfg["loop"]
    case = Case(tmp_path, cfg, seed=8)
    toks = tokens_of(cfg, 30, 1)
    rp = case.replay("float32")
    try:
        run_schedule(rp, case, {"a": toks}, [[("a", 12)], [("a", 18)]], "float32")
    finally:
        rp.close()


# ----------------------------------------------------------------------------------------------------- the engine's own entry point
def test_greedy_generation_through_the_engine(loop_case):
    """LLM.generate with temperature 0 (scheduler, chunked prefill, captured graphs, sampling kernel) against greedy decoding of
    the reference."""
    from nanovllm import LLM, SamplingParams
    prompts = [tokens_of(CFG_LOOP, n, 50 + n) for n in (5, 40, 17)]
    llm = LLM(loop_case.path, dtype="float32", max_num_seqs=4, max_num_batched_tokens=32, max_model_len=128, num_kvcache_blocks=6,
              chunked_prefill=True)
    try:
        assert llm.model_runner.graphs, "one-token steps are expected to replay captured graphs"
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True), use_tqdm=False)
    finally:
        llm.exit()
    for prompt, out in zip(prompts, outs):
        toks = list(prompt)
        for _ in range(12):
            toks.append(int(R.forward(loop_case.W, CFG_LOOP, toks)[-1].argmax()))
        assert out["token_ids"] == toks[len(prompt):]


def test_pool_sized_by_the_engine_with_and_without_attention_layers(tmp_path, loop_case):
    """No page count given: the engine sizes the pool from free memory less the state pools; a model of recurrent mixers only
    keeps no pages at all and gets a count that merely bounds the tokens."""
    from nanovllm import LLM, SamplingParams
    cfg = config([GLA_A, HGRN_B], width=64, vocab=40)
    recurrent_only = Case(tmp_path, cfg, seed=8)
    for case, c in ((recurrent_only, cfg), (loop_case, CFG_LOOP)):
        prompt = tokens_of(c, 9, 3)
        llm = LLM(case.path, dtype="float32", max_num_seqs=3, max_num_batched_tokens=64, max_model_len=300, gpu_memory_utilization=0.2)
        try:
            pages = llm.model_runner.config.num_kvcache_blocks
            assert pages == 3 * 2 if case is recurrent_only else pages > 100
            out = llm.generate([prompt], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True), use_tqdm=False)[0]
        finally:
            llm.exit()
        toks = list(prompt)
        for _ in range(4):
            toks.append(int(R.forward(case.W, c, toks)[-1].argmax()))
        assert out["token_ids"] == toks[len(prompt):]


def test_captured_decode_steps_match_eager_ones(loop_case):
    """One-token steps replayed from the captured graph (routing, expert tiles and states inside it) against the same steps
    run eagerly: several replays, with eager work between them."""
    from nanovllm.config import Config
    from nanovllm.engine.model_runner import ModelRunner
    from nanovllm.engine.sequence import Sequence
    toks = [tokens_of(CFG_LOOP, n, 70 + n) for n in (30, 11, 21)]
    logits = {}
    for eager in (True, False):
        cfg = Config(loop_case.path, max_num_batched_tokens=64, max_num_seqs=4, max_model_len=128, num_kvcache_blocks=6, num_state_slots=4,
                     chunked_prefill=True, enforce_eager=eager, async_scheduling=False, dtype="float32")
        runner = ModelRunner(cfg, 0, [])
        try:
            seqs = []
            for i, t in enumerate(toks):
                s = Sequence(list(t[:-6]))
                s.block_table, s.state_slot, s.num_new_tokens = [i], i, len(t) - 6
                seqs.append(s)
            runner.forward_logits(seqs)
            rows = []
            for step in range(6):
                for s, t in zip(seqs, toks):
                    s.num_cached_tokens += s.num_new_tokens
                    s.append_token(t[len(t) - 6 + step])
                    s.num_new_tokens = 1
                out, _, _ = runner.forward_logits(seqs)
                rows.append(out.float().cpu().numpy())
            logits[eager] = np.stack(rows)
            assert eager or runner.graphs
        finally:
            runner.exit()
    assert np.abs(logits[True] - logits[False]).max() < 1e-4 * np.abs(logits[True]).max()
    for i, t in enumerate(toks):
        want = loop_case.ref(t)
        for step in range(6):
            assert rel_err(logits[False][step, i:i + 1], want[len(t) - 6 + step:len(t) - 5 + step]) < TOL["float32"]
