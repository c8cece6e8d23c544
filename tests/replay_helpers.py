"""Builds traces (lists of steps) for the replay tests and collects the logits
they produce, keyed by (request, position), so that every way of cutting the
same requests can be compared with the plain implementation row by row."""

from __future__ import annotations

import numpy as np
import torch

import plain_llama
from tokasaurus_amd.engine.batch import StepEntry


def plain_rows(folder, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    cfg, w = plain_llama.load_folder(folder)
    return {rid: plain_llama.forward_logits(cfg, w, toks) for rid, toks in requests.items()}


def run_steps(runner, steps: list[dict]) -> dict[tuple[str, int], torch.Tensor]:
    """steps: [{"entries": [(id, tokens, want)], "end": [ids]}]; returns logits by
    (request id, absolute position)."""
    got: dict[tuple[str, int], torch.Tensor] = {}
    held: dict[str, int] = {}
    for step in steps:
        entries = [StepEntry(rid, list(toks), list(want)) for rid, toks, want in step["entries"]]
        logits = runner.step(entries).float().cpu()
        row = 0
        for rid, toks, want in step["entries"]:
            start = held.get(rid, 0)
            for w in want:
                got[(rid, start + w)] = logits[row]
                row += 1
            held[rid] = start + len(toks)
        assert row == logits.shape[0]
        for rid in step.get("end", []):
            runner.release(rid)
            held.pop(rid, None)
        runner.manager.check()
    return got


def whole(rid: str, tokens: list[int]) -> list[dict]:
    return [{"entries": [(rid, tokens, list(range(len(tokens))))], "end": [rid]}]


def tail_one_by_one(rid: str, tokens: list[int], tail: int = 32) -> list[dict]:
    head = len(tokens) - tail
    steps = [{"entries": [(rid, tokens[:head], list(range(head)))]}]
    for i in range(head, len(tokens)):
        steps.append({"entries": [(rid, [tokens[i]], [0])]})
    steps[-1]["end"] = [rid]
    return steps


def portions(rid: str, tokens: list[int], sizes: list[int]) -> list[dict]:
    steps, at, k = [], 0, 0
    while at < len(tokens):
        n = min(sizes[k % len(sizes)], len(tokens) - at)
        steps.append({"entries": [(rid, tokens[at : at + n], list(range(n)))]})
        at += n
        k += 1
    steps[-1]["end"] = [rid]
    return steps


def mixed_trace(reqs: dict[str, list[int]], seed: int, max_live: int = 4):
    """Up to four live requests; portions of some beside single tokens of others; a
    request may sit out a step; finished requests' pages go to later ones."""
    rng = np.random.default_rng(seed)
    waiting = list(reqs)
    live: dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            live[waiting.pop(0)] = 0
        entries, ended = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step
            at, toks = live[rid], reqs[rid]
            left = len(toks) - at
            n = 1 if (left <= 12 or rng.random() < 0.4) else int(rng.choice([2, 3, 5, 8, 13, 21]))
            n = min(n, left)
            entries.append((rid, toks[at:at + n], list(range(n))))
            live[rid] = at + n
            if live[rid] == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"entries": entries, "end": ended})
    return steps


def compare(got, want_rows: dict[str, torch.Tensor], atol: float, rtol: float) -> float:
    """Every collected row against the plain row; returns the largest error seen.
    On a mismatch, names the first wrong (request, position)."""
    worst = 0.0
    for (rid, pos), row in sorted(got.items()):
        ref = want_rows[rid][pos]
        err = (row - ref).abs()
        bound = atol + rtol * ref.abs()
        if not bool((err <= bound).all()):
            i = int((err - bound).argmax())
            raise AssertionError(
                f"request {rid} position {pos}: logit {i} is {row[i].item():.6f}, plain {ref[i].item():.6f} "
                f"(error {err[i].item():.3e}, allowed {bound[i].item():.3e})"
            )
        worst = max(worst, float(err.max()))
    return worst


def compare_with_bfloat16_measure(got, plain: dict[str, torch.Tensor], plain16: dict[str, torch.Tensor],
                                  atol: float, rtol: float) -> float:
    """For models wider than the tiny ones, whose rounding errors outgrow a fixed bound: a
    row of bfloat16 logits passes when it is within the bound, or else when it is less than
    twice as far from the plain 32-bit row (root mean square) as the plain model computing
    in bfloat16 is.  A wrong key or page moves a row many times further than rounding does.
    Returns the largest ratio seen among the rows beyond the bound (0 if none)."""
    worst = 0.0
    for (rid, pos), row in sorted(got.items()):
        ref = plain[rid][pos]
        err = (row - ref).double()
        if bool((err.abs() <= atol + rtol * ref.abs()).all()):
            continue
        err16 = (plain16[rid][pos] - ref).double()
        ratio = float(err.pow(2).mean().sqrt() / err16.pow(2).mean().sqrt().clamp_min(1e-12))
        if ratio >= 2.0:
            raise AssertionError(f"request {rid} position {pos}: {ratio:.2f} times as far from the plain logits as "
                                 f"the plain model in bfloat16 (largest error {float(err.abs().max()):.3e})")
        worst = max(worst, ratio)
    return worst


# --------------------------------------------------------------------------
# faults put in on purpose: what the comparisons above must find
# --------------------------------------------------------------------------


def swap_pages(runner, rid_a: str, block_a: int, rid_b: str, block_b: int, group: int = 0) -> None:
    """Exchange one page between the block tables of two live requests: every read stays
    inside pages that the two own, but request a now sees a page of b's keys and values in
    place of its own (and the other way round)."""
    m = runner.manager
    ra, rb = m.requests[rid_a], m.requests[rid_b]
    pa, pb = ra.tables[group][block_a], rb.tables[group][block_b]
    assert pa >= 0 and pb >= 0 and pa != pb
    ra.tables[group][block_a], rb.tables[group][block_b] = pb, pa
    if m.slot_tables is not None:
        m.slot_tables[group][ra.slot, block_a] = pb
        m.slot_tables[group][rb.slot, block_b] = pa


def shift_position(runner, rid: str) -> None:
    """The request's next token is taken to stand one position further than it does: it is
    rotated for the wrong place and its key lands one slot too far, leaving a slot of zeros."""
    rc = runner.manager.requests[rid]
    runner.manager.reserve(rid, rc.num_tokens + 2)
    rc.num_tokens += 1


def faulty_tail(runner, reqs: dict[str, list[int]], victim: str, tail: int, fault) -> dict[tuple[str, int], torch.Tensor]:
    """Every request's tokens but the victim's last ``tail`` go in honestly and unobserved; then
    ``fault(runner)`` is applied and the victim's last tokens are decoded one by one.  Returns
    their logits keyed as the plain rows are, (request, position the token truly has)."""
    for rid, toks in reqs.items():
        n = len(toks) - tail if rid == victim else len(toks)
        runner.step([StepEntry(rid, toks[:n], [])])
    fault(runner)
    toks = reqs[victim]
    got = {}
    for pos in range(len(toks) - tail, len(toks)):
        got[(victim, pos)] = runner.step([StepEntry(victim, [toks[pos]], [0])]).float().cpu()[0]
    for rid in reqs:
        runner.release(rid)
    return got
