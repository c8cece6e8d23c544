"""Per-request sampling options.

The reference samples with a temperature only: ``top_p`` must be 1.0
(tokasaurus/model/types.py:318, tokasaurus/model/llama.py:469) and penalties,
logit bias and best_of are rejected (tokasaurus/server/utils.py:459-531).
Temperature 0 is greedy (tokasaurus/model/types.py:302-312).  The reference
ignores a request's seed (tokasaurus/server/types.py:36); here it selects the
request's stream of uniform numbers.  ``topk_logprobs`` asks for the most probable
tokens of every step and their log-probabilities (tokasaurus/server/types.py:151),
at most as many as the engine's ``max_topk_logprobs``.
"""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_p: float = 1.0
    max_tokens: int = 16
    ignore_eos: bool = False
    seed: int | None = None
    topk_logprobs: int | None = None

    def __post_init__(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if self.top_p != 1.0:
            raise ValueError("top_p other than 1.0 is not supported")
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if self.topk_logprobs is not None and self.topk_logprobs < 1:
            raise ValueError("topk_logprobs must be at least 1")
