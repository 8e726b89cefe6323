"""Per-request sampling options (front-end contract of the reference's sampling_params.py:19-45)."""
from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0
    max_tokens: int = 64
    ignore_eos: bool = False

    def __post_init__(self):
        # temperature 0 selects the most likely token (the sampler's race runs without noise for such a row; the
        # reference forbids it); anything between 0 and 1e-10 would overflow logits / T
        assert self.temperature == 0 or self.temperature > 1e-10, "temperature must be 0 (greedy) or above 1e-10"
