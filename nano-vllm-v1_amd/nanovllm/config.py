"""Engine configuration: the twelve fields (names and defaults) of the reference's config.py:53-64, plus
``async_scheduling`` (not in the reference; ON by default): the engine schedules and launches step n+1 before it has
read step n's sampled ids, so the GPU never waits for the host between steps.  Same tokens as the synchronous loop up
to what depends on WHEN a value is seen (eos ends a sequence one step later: the token computed past it is dropped);
``async_scheduling=False`` runs the reference's loop (engine/llm_engine.py:117-126): schedule, run, read ids, postprocess.

``dtype`` and ``num_state_slots`` are not in the reference either: the activation type a model is served in (models
that support fp32 run every product in true 32-bit then) and the number of recurrent-state slots.

``model`` is a local directory holding a Hugging Face ``config.json`` (and optionally
``*.safetensors`` weights; without them the runner initialises synthetic weights).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from types import SimpleNamespace

import torch


def load_hf_config(path: str):
    """config.json of a model directory.  A config that names a `model_type` goes through transformers' AutoConfig when it
    is importable; any other (a design that no library knows: it names its `architecture` itself) is the raw JSON as a
    namespace, nested objects left as dicts."""
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    if "model_type" in raw:
        try:
            from transformers import AutoConfig
            return AutoConfig.from_pretrained(path)
        except ImportError:
            pass
    if isinstance(raw.get("torch_dtype"), str):
        raw["torch_dtype"] = getattr(torch, raw["torch_dtype"])
    return SimpleNamespace(**raw)


def model_dtype(hf_config) -> torch.dtype:
    dt = getattr(hf_config, "dtype", None) or getattr(hf_config, "torch_dtype", None) or torch.bfloat16
    return getattr(torch, dt) if isinstance(dt, str) else dt


@dataclass
class Config:
    model: str
    max_num_batched_tokens: int = 16384
    max_num_seqs: int = 512
    max_model_len: int = 40960
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1
    enforce_eager: bool = False
    hf_config: object | None = None
    eos: int = -1
    kvcache_block_size: int = 256
    num_kvcache_blocks: int = -1
    chunked_prefill: bool = False
    async_scheduling: bool = True
    dtype: str | None = None            # "bfloat16" / "float32": serve the model in this type instead of its checkpoint's (None)
    num_state_slots: int = -1           # recurrent-state slots (models with a per-sequence state); -1: one per max_num_seqs
    prefix_caching: bool = True         # share resident pages between prompts with a common prefix (off for recurrent models)
    recurrent_state: bool = False       # set by the runner: the loaded model keeps a state per sequence

    def __post_init__(self):
        # the reference asserts a multiple of 256 (config.py:82) but its Sequence.block_size is the constant 256
        # (engine/sequence.py:73) and every kernel here indexes 256-token pages: any other size would read wrong keys
        assert self.kvcache_block_size == 256, "the KV page is 256 tokens (kvcache_block_size must stay 256)"
        assert 1 <= self.tensor_parallel_size <= 8
        if self.hf_config is None:
            self.hf_config = load_hf_config(self.model)
        # (a design whose positions no table bounds names neither max_position_embeddings nor max_positions: max_model_len stands as given)
        bound = getattr(self.hf_config, "max_position_embeddings", None) or getattr(self.hf_config, "max_positions", None)
        self.max_model_len = min(self.max_model_len, int(bound) if bound else self.max_model_len)
        if self.num_state_slots <= 0:
            self.num_state_slots = self.max_num_seqs
