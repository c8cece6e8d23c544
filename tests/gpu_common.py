"""Shared by the GPU tests: model folders made once per session, tolerances."""

from __future__ import annotations

import pytest

import plain_llama
from tiny_models import TINY, make_folder
from tokasaurus_amd.sampling import uniform_for

# Logits of the tiny models are of order 1.  In 32-bit the engine and the plain
# implementation differ by the order of summation only.  In bfloat16 every
# activation is rounded to 8 bits of mantissa on its way through two or three
# blocks, which moves logits by about a percent of their scale.
TOL = {
    "float32": dict(atol=5e-5, rtol=1e-4),
    "bfloat16": dict(atol=6e-2, rtol=5e-2),
}


@pytest.fixture(scope="session")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_folder(root / name, cfg, seed=11 + i) for i, (name, (cfg, _)) in enumerate(sorted(TINY.items()))}


def plain_generate(folder, prompt, max_tokens, temperature=0.0, engine_seed=0, request_seed=0, eos=()):
    """Token by token with the whole sequence recomputed; the same uniform numbers as the engine draws."""
    cfg, w = plain_llama.load_folder(folder)
    ids, out, lps = list(prompt), [], []
    for i in range(max_tokens):
        logits = plain_llama.forward_logits(cfg, w, ids)[-1]
        u = uniform_for(engine_seed, request_seed, i) if temperature > 0 else 0.0
        tok, lp = plain_llama.sample(logits, temperature, u)
        out.append(tok)
        lps.append(lp)
        ids.append(tok)
        if tok in eos:
            break
    return out, lps


def check_token_follows_plain(logits, tok: int, temperature: float, u: float, slack: float = 0.0) -> None:
    """A token the bfloat16 engine chose, judged against the plain 32-bit logits of the same
    history: rounding may flip a near tie but no more.  Greedy: the token's plain logit is within
    0.08 (+ slack) of the best.  Sampled with the uniform number u: u lies within 0.05 (+ slack)
    of the token's interval of cumulative plain probability (rounding moves the intervals' edges
    by a few hundredths at most; a wrong distribution moves them anywhere)."""
    import torch

    if temperature == 0:
        gap = float(logits.max() - logits[tok])
        assert gap < 0.08 + slack, f"token {tok} is {gap:.3f} below the plain best {int(logits.argmax())}"
        return
    p = torch.softmax(logits.double() / temperature, -1)
    hi = float(p[: tok + 1].sum())
    lo = hi - float(p[tok])
    tol = 0.05 + slack
    assert lo - tol <= u <= hi + tol, f"token {tok} covers [{lo:.4f}, {hi:.4f}) of the plain distribution, u = {u:.4f}"
