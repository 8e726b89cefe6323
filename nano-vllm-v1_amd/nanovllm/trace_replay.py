"""Replay of a recorded schedule: the caller dictates, step by step, which tokens of which request run together, and
reads back logits at any of their positions.  Used by bin/trace_run and by tests that pin the engine's numerics
against a schedule (whole prompts, prompts cut into portions, decoding, mixed batches, pages and slots used again).

Nothing here computes: requests are the engine's `Sequence`s, pages and state slots come from the scheduler's
`BlockManager` (`Scheduler.replay_step`), and a step is `ModelRunner.forward_logits(seqs, rows=...)` - the same
flattening, kernels, caches and state pools that `LLMEngine.generate` drives; only the scheduler's own choice of what
to run is replaced by the trace's.
"""
from __future__ import annotations

import json

import numpy as np
import torch

from . import _hip
from .config import Config
from .engine.model_runner import ModelRunner
from .engine.scheduler import Scheduler


class UnsupportedDtype(Exception):
    pass


class TraceReplay:
    def __init__(self, model: str, dtype: str = "bfloat16", max_tokens: int = 4096, state_slots: int = 4, **config):
        """`max_tokens`: the most tokens live requests hold at any time (the page pool is sized for it, each request
        rounded up to whole pages); `state_slots`: the most requests live at a time."""
        page = 256
        blocks = -(-max_tokens // page) + state_slots             # every live request may leave one page partly used
        cfg = dict(max_num_seqs=state_slots, num_state_slots=state_slots, num_kvcache_blocks=blocks,
                   max_model_len=max_tokens + 1, max_num_batched_tokens=max(min(max_tokens, 8192), 1), enforce_eager=True,
                   async_scheduling=False, chunked_prefill=True, dtype=dtype)
        cfg.update(config)
        self.config = Config(model, **cfg)
        try:
            self.runner = ModelRunner(self.config, 0, [])
        except _hip.HipError as e:
            if "unsupported by" in str(e):
                raise UnsupportedDtype(str(e)) from None
            raise
        self.scheduler = Scheduler(self.config)
        self.live: dict = {}

    def step(self, entries: list[dict], end: list | tuple = ()) -> np.ndarray | None:
        """Run one step; returns fp32 logits [wanted, vocab] (None when no entry wants any)."""
        seqs, rows, offset = [], [], 0
        for e in entries:
            seqs.append(self.scheduler.replay_step(self.live, e["id"], e["tokens"]))
            rows += [offset + int(w) for w in e.get("want", ())]
            offset += len(e["tokens"])
        logits = None
        if seqs:
            out, _, _ = self.runner.forward_logits(seqs, rows=np.asarray(rows, dtype=np.int32))
            if rows:
                logits = out.float().cpu().numpy()
            self.scheduler.replay_done(seqs)
        for rid in end:
            self.scheduler.replay_end(self.live, rid)
        return logits

    def step_line(self, line: str):
        msg = json.loads(line)
        return msg["step"], self.step(msg["entries"], msg.get("end", ()))

    def close(self):
        if self.runner is not None:
            torch.cuda.synchronize()
            self.runner.exit()
            self.runner = None
