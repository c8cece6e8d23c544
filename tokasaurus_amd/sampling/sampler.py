"""Greedy and temperature sampling over the step's logits
(tokasaurus/model/llama.py:377-423).

Rows with temperature 0 take the largest raw logit; the others draw from
softmax(logits / T) by inverse CDF with one uniform number per row.  The
reference takes that number from the global generator (llama.py:365); here it is
a pure function of (engine seed, request seed, index of the token in the
completion), so a request's tokens do not depend on what else was in the batch
and a request that is restarted draws the same tokens again.  The kernels are
``ops.sample`` and ``ops.topk_logprobs``; the step function calls them with the step's rows.
"""

from __future__ import annotations

_MASK = (1 << 64) - 1


def _mix(x: int) -> int:
    """splitmix64 finaliser."""
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform_for(engine_seed: int, request_seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits, fixed by its three arguments."""
    h = _mix(_mix(_mix(engine_seed & _MASK) ^ (request_seed & _MASK)) ^ (index & _MASK))
    return (h >> 40) / float(1 << 24)
