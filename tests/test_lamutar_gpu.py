"""Lamutar through the engine against the plain fp32 restatement in tests/lamutar_reference.py.

Every test makes its own small configuration and random weights (written as config.json + model.safetensors into a
temporary directory, so the config reader and the loader are part of what is tested), runs a schedule through
nanovllm.trace_replay.TraceReplay (the engine's runner, page/state manager and kernels) and compares logits - and, for
single layers, the residual stream - with the reference run over each whole sequence.  fp32 serving is compared
tightly, bf16 serving within the rounding of its products.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

import lamutar_reference as R

pytestmark = pytest.mark.gpu

ATTN_A = {"type": "attention", "mixer": {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.3,
                                         "rot": {"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}}},
          "mlp": {"kind": "dense", "ff": 100}}
ATTN_B = {"type": "attention", "mixer": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 16, "scale": 0.25,
                                         "rot": {"base": 500.0, "dims": 16, "scaling": None}}, "mlp": None}
DELTA_A = {"type": "general_delta", "mixer": {"heads": 3, "dim": 20}, "mlp": {"kind": "dense", "ff": 60}}
DELTA_B = {"type": "general_delta", "mixer": {"heads": 2, "dim": 32}, "mlp": None}

CFG_LOOP = {"architecture": "Lamutar", "vocab": 131, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 7.5,
            "loop": {"start": 1, "stop": 3, "times": 3}, "layers": [DELTA_A, ATTN_A, DELTA_B, ATTN_B]}
CFG_FLAT = {"architecture": "Lamutar", "vocab": 200, "width": 128, "norm": {"eps": 1e-6}, "logit_softcap": None, "loop": None,
            "layers": [{"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 128, "vdim": 64, "scale": 0.09,
                                                       "rot": {"base": 1e6, "dims": 64, "scaling": {"factor": 3.0, "original": 256, "fast": 24.0, "slow": 2.0}}},
                        "mlp": {"kind": "dense", "ff": 256}},
                       {"type": "general_delta", "mixer": {"heads": 2, "dim": 64}, "mlp": {"kind": "dense", "ff": 256}}]}


def random_weights(cfg: dict, seed: int, ranks=(8, 24)) -> dict:
    """bf16 weights in checkpoint naming; decay offsets spread so that some channels forget fast and some hardly at all."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    W = {}

    def mat(name, out, inp, scale=None):
        W[name] = torch.randn(out, inp, generator=g) * (scale if scale is not None else 1.0 / math.sqrt(inp))

    def norm(name):
        W[name] = 1.0 + 0.2 * torch.randn(D, generator=g)
        W[name + ".b"] = 0.1 * torch.randn(D, generator=g)
        W[name + ".alpha"] = torch.tensor(0.4 + 0.4 * torch.rand((), generator=g).item())

    mat("embed", V, D, 1.0)
    mat("head", V, D)
    norm("final.norm")
    if cfg.get("loop"):
        mat("loop.in", D, 2 * D, 1.0 / math.sqrt(D))
        W["loop.step"] = 0.3 * torch.randn(cfg["loop"]["times"], D, generator=g)
    n_delta = 0
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if L.get("mlp") else ()):
            norm(p + nm)
        h, d = m["heads"], m["dim"]
        if L["type"] == "attention":
            gk, dv = m.get("kv_heads", h), m.get("vdim", d)
            mat(p + "mix.q", h * d, D)
            mat(p + "mix.k", gk * d, D)
            mat(p + "mix.v", gk * dv, D)
            mat(p + "mix.g", h, D)
            W[p + "mix.q.norm"] = 1.0 + 0.2 * torch.randn(h * d, generator=g)
            W[p + "mix.k.norm"] = 1.0 + 0.2 * torch.randn(gk * d, generator=g)
            mat(p + "mix.o", D, h * dv)
        else:
            n, rank = h * d, ranks[n_delta % len(ranks)]
            n_delta += 1
            for leaf in ("r", "k", "v", "a", "g"):
                mat(p + "mix." + leaf, n, D)
            mat(p + "mix.w1", rank, D)
            mat(p + "mix.w2", n, rank, 0.5)
            W[p + "mix.w0"] = -6.0 + 7.0 * torch.rand(n, generator=g)
            W[p + "mix.a.b"] = torch.randn(n, generator=g)
            W[p + "mix.norm"] = 1.0 + 0.2 * torch.randn(n, generator=g)
            mat(p + "mix.o", D, n)
        if L.get("mlp"):
            mat(p + "mlp.gate", L["mlp"]["ff"], D)
            mat(p + "mlp.up", L["mlp"]["ff"], D)
            mat(p + "mlp.down", D, L["mlp"]["ff"])
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def write_model(path, cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


class Case:
    """A model on disk, its reference weights in fp32 and cached reference logits per token list."""

    def __init__(self, tmp, cfg, seed=0, weights=None):
        self.cfg = cfg
        w = weights if weights is not None else random_weights(cfg, seed)
        self.path = write_model(tmp, cfg, w)
        self.W = {k: v.float() for k, v in w.items()}
        self._ref = {}

    def ref(self, tokens):
        key = tuple(tokens)
        if key not in self._ref:
            self._ref[key] = R.forward(self.cfg, self.W, list(tokens)).numpy()
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
    return Case(tmp_path_factory.mktemp("lamutar_loop"), CFG_LOOP, seed=1)


@pytest.fixture(scope="module")
def flat_case(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("lamutar_flat"), CFG_FLAT, seed=2)


def run_schedule(rp, case, requests: dict, schedule: list, dtype: str):
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
            assert err < TOL[dtype], f"request {rid} tokens {lo}..{hi}: error {err:.3g}"
            worst = max(worst, err)
            row += hi - lo
    assert all(at[r] == len(requests[r]) for r in requests)
    return worst


# ----------------------------------------------------------------------------------------------------- single mechanisms
@pytest.mark.parametrize("layer", [ATTN_A, ATTN_B, DELTA_A, DELTA_B], ids=["attention+ff", "attention(full rotary, no gqa)", "delta+ff", "delta"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_stream_matches(tmp_path, layer, dtype):
    """One layer of each kind, no loop: the residual stream after it and the logits."""
    cfg = {"architecture": "Lamutar", "vocab": 50, "width": 72, "norm": {"eps": 1e-5}, "logit_softcap": 5.0, "loop": None, "layers": [layer]}
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
    want = R.forward(cfg, case.W, toks, col).numpy()
    assert np.abs(stream - col[0].numpy()).max() < (1e-4 if dtype == "float32" else 0.15) * max(1.0, float(col[0].abs().max()))
    assert rel_err(got, want) < TOL[dtype]


def test_loop_passes_keep_separate_caches_and_states(loop_case):
    """A looped span (three passes over an attention and a delta layer): every layer run against the reference."""
    toks = tokens_of(CFG_LOOP, 40, 7)
    rp = loop_case.replay("float32")
    try:
        rp.runner.model.collect = []
        rp.step([{"id": 0, "tokens": toks, "want": [0]}], [0])
        streams = [c.cpu().numpy() for c in rp.runner.model.collect]
    finally:
        rp.close()
    col = []
    R.forward(CFG_LOOP, loop_case.W, toks, col)
    assert len(streams) == len(col) == 1 + 2 * 3 + 1
    for n, (a, b) in enumerate(zip(streams, col)):
        assert np.abs(a - b.numpy()).max() < 2e-4 * max(1.0, float(b.abs().max())), f"layer run {n}"


def test_linear_any_ragged_shapes_both_types():
    from nanovllm import ops
    g = torch.Generator().manual_seed(0)
    for m, n, k in [(1, 5, 3), (7, 64, 64), (65, 131, 96), (130, 66, 17), (3, 976, 320), (33, 8, 200)]:
        x, w, b = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g), torch.randn(n, generator=g)
        want32 = x @ w.t() + b
        y = ops.linear_any(x.cuda(), w.cuda(), b.cuda())
        assert y.dtype == torch.float32 and (y.cpu() - want32).abs().max() < 1e-4 * k ** 0.5
        xb, wb = x.bfloat16(), w.bfloat16()
        want16 = xb.float() @ wb.float().t()
        y = ops.linear_any(xb.cuda(), wb.cuda(), None, out_f32=True)
        assert (y.cpu() - want16).abs().max() < 1e-3 * k ** 0.5, (m, n, k)
        y = ops.linear_any(xb.cuda(), wb.cuda())
        assert y.dtype == torch.bfloat16 and (y.float().cpu() - want16).abs().max() < 0.02 * max(1.0, float(want16.abs().max()))


def test_rows_of_a_product_do_not_depend_on_the_batch():
    """The same row alone and among others: identical bits (the any-shape kernel) in both types."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(1)
    x, w = torch.randn(150, 100, generator=g).cuda(), torch.randn(77, 100, generator=g).cuda()
    for cast in (torch.float32, torch.bfloat16):
        xa, wa = x.to(cast), w.to(cast)
        full = ops.linear_any(xa, wa, None, out_f32=True)
        for r in (0, 63, 64, 149):
            assert torch.equal(ops.linear_any(xa[r:r + 1].contiguous(), wa, None, out_f32=True)[0], full[r])


# ----------------------------------------------------------------------------------------------------- schedules
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_then_token_by_token(loop_case, dtype):
    toks = tokens_of(CFG_LOOP, 90, 11)
    rp = loop_case.replay(dtype)
    try:
        run_schedule(rp, loop_case, {"a": toks}, [[("a", 50)]] + [[("a", 1)]] * 40, dtype)
        # the first tokens of a sequence, one by one from the very start
        run_schedule(rp, loop_case, {"b": toks[:12]}, [[("b", 1)]] * 12, dtype)
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
    """Delta-rule layers only: one piece, portions and single tokens give identical logits (one summation order)."""
    cfg = {"architecture": "Lamutar", "vocab": 64, "width": 64, "norm": {"eps": 1e-6}, "logit_softcap": None, "loop": None,
           "layers": [DELTA_A, DELTA_B]}
    case = Case(tmp_path, cfg, seed=5)
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
    the first two runs on pages and slots that others have left behind, some of them longer than what was there."""
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
    """Portions that end one token before, at and after a page border; decoding across it; a second page border."""
    toks = tokens_of(CFG_FLAT, 530, 41)
    rp = flat_case.replay(dtype, max_tokens=1100)
    try:
        run_schedule(rp, flat_case, {"a": toks}, [[("a", 255)], [("a", 1)], [("a", 1)], [("a", 2)], [("a", 251)], [("a", 3)]] + [[("a", 1)]] * 17, dtype)
        run_schedule(rp, flat_case, {"b": toks[:300]}, [[("b", 256)], [("b", 44)]], dtype)
    finally:
        rp.close()


def test_long_decoding(flat_case):
    toks = tokens_of(CFG_FLAT, 330, 43)
    rp = flat_case.replay("float32", max_tokens=512)
    try:
        run_schedule(rp, flat_case, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 325, "float32")
    finally:
        rp.close()


# ----------------------------------------------------------------------------------------------------- faults that random weights would hide
def sharp_attention_case(tmp, value_rotation_matters=True):
    """An attention-only model whose keys equal its queries (same weights, no rotary dimensions worth speaking of) and
    whose scale is large: a query puts nearly all its weight on the earlier occurrence of its own token, wherever it is."""
    layer = {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 1.0,
                                            "rot": {"base": 1e4, "dims": 2, "scaling": None}}, "mlp": None}
    cfg = {"architecture": "Lamutar", "vocab": 700, "width": 64, "norm": {"eps": 1e-6}, "logit_softcap": None, "loop": None, "layers": [layer]}
    w = random_weights(cfg, 9)
    w["l0.mix.k"] = w["l0.mix.q"].clone()
    w["l0.mix.k.norm"] = w["l0.mix.q.norm"].clone()
    w["l0.mix.v"] = w["l0.mix.v"] * 4
    return Case(tmp, cfg, weights=w), cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_decides_the_output(tmp_path, dtype):
    case, cfg = sharp_attention_case(tmp_path)
    n = 600
    base = list(range(1, n + 1))                       # all tokens distinct ...
    for far in (0, 3, 255, 256, 257, 511, 512):        # ... except the last, which repeats the one at `far`
        toks = base[:n - 1] + [base[far]]
        other = base[:n - 1] + [699]
        ref, ref_other = case.ref(toks)[-1:], case.ref(other)[-1:]
        assert rel_err(ref_other, ref) > 0.3           # the far key matters: without it the logits are others
        rp = case.replay(dtype, max_tokens=1300)
        try:
            whole = rp.step([{"id": 0, "tokens": toks, "want": [n - 1]}], [0])
            rp.step([{"id": 1, "tokens": toks[:n - 1], "want": []}])
            decoded = rp.step([{"id": 1, "tokens": toks[n - 1:], "want": [0]}], [1])
        finally:
            rp.close()
        tol = TOL[dtype] if dtype == "float32" else 0.15      # (sharp weights magnify the rounding of bf16 scores)
        assert rel_err(whole, ref) < tol and rel_err(decoded, ref) < tol, far


def test_delta_state_carries_a_token_from_far_back(tmp_path):
    """Decay offsets near -9 keep a channel's memory for hundreds of tokens: the first token still shapes the last logits,
    and a state that were lost or reset between portions would show."""
    cfg = {"architecture": "Lamutar", "vocab": 90, "width": 48, "norm": {"eps": 1e-6}, "logit_softcap": None, "loop": None,
           "layers": [{"type": "general_delta", "mixer": {"heads": 2, "dim": 16}, "mlp": None}]}
    w = random_weights(cfg, 4)
    w["l0.mix.w0"] = torch.full_like(w["l0.mix.w0"], -9.0)
    w["l0.mix.a.b"] = torch.full_like(w["l0.mix.a.b"], -6.0)
    case = Case(tmp_path, cfg, weights=w)
    toks = tokens_of(cfg, 400, 8)
    changed = [(toks[0] + 1) % 90] + toks[1:]
    assert rel_err(case.ref(changed)[-1:], case.ref(toks)[-1:]) > 20 * TOL["float32"]      # 400 tokens later it still shows
    rp = case.replay("float32", max_tokens=1024)
    try:
        run_schedule(rp, case, {"a": toks}, [[("a", 100)], [("a", 156)], [("a", 1)], [("a", 140)], [("a", 2)], [("a", 1)]], "float32")
    finally:
        rp.close()


# ----------------------------------------------------------------------------------------------------- the engine's own entry point
def test_greedy_generation_through_the_engine(loop_case):
    """LLM.generate with temperature 0 (scheduler, chunked prefill, sampling kernel) against greedy decoding of the reference."""
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
            toks.append(int(R.forward(CFG_LOOP, loop_case.W, toks)[-1].argmax()))
        assert out["token_ids"] == toks[len(prompt):]


def test_temperature_zero_rows_take_the_maximum():
    """Rows with temperature 0 beside sampled rows in one sampler call: the greedy rows are the row maxima (lowest index
    among equals), whatever the seed."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(6, 1000, generator=g)
    logits[2, 17] = logits[2, 500] = 9.0                      # a tie: the lower index wins
    temps = torch.tensor([0.0, 1.0, 0.0, 0.7, 0.0, 0.0])
    for dtype in (torch.float32, torch.bfloat16):
        lg = logits.to(dtype).cuda()
        for seed in (1, 2):
            ids = ops.sample(lg, temps.cuda(), seed, 5).cpu()
            want = lg.float().cpu().argmax(-1)
            for r in (0, 4, 5):
                assert ids[r] == want[r]
            assert ids[2] == 17


def test_sizes_no_kernel_tile_divides(tmp_path):
    """A delta head size that is no multiple of 4, a width that is no multiple of 8, an odd decay rank, one KV head, and
    attention heads of 256 (the largest the kernels take; fp32 serving needs more than the default 64 KB of LDS there)."""
    cfg = {"architecture": "Lamutar", "vocab": 37, "width": 50, "norm": {"eps": 1e-6}, "logit_softcap": 3.0,
           "loop": {"start": 0, "stop": 2, "times": 1},
           "layers": [{"type": "general_delta", "mixer": {"heads": 3, "dim": 10}, "mlp": {"kind": "dense", "ff": 34}},
                      {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 256, "vdim": 256, "scale": 0.05,
                                                      "rot": {"base": 777.0, "dims": 256, "scaling": {"factor": 8.0, "original": 32, "fast": 4.0, "slow": 0.5}}},
                       "mlp": None}]}
    case = Case(tmp_path, cfg, weights=random_weights(cfg, 6, ranks=(5,)))
    toks = tokens_of(cfg, 80, 3)
    for dtype in ("float32", "bfloat16"):
        rp = case.replay(dtype)
        try:
            run_schedule(rp, case, {"a": toks, "b": toks[:7]}, [[("a", 33), ("b", 5)], [("a", 1), ("b", 2)], [("a", 46)]], dtype)
        finally:
            rp.close()
