"""Trace replay: feeds given token ids through the model step by step and writes
logits.  It samples nothing and has no forward pass, cache or loader of its
own: it drives the ``ModelRunner`` that generation uses.

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits at
the wanted places as little-endian float32 [wanted, vocab], and ``<out>/<step>.json``
names the rows: ``{"step": s, "vocab": V, "rows": [[request id, position], ...]}``, the
position being the token's place in its request counted from 0.  After every step
the line ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

import numpy as np

from tokasaurus_amd.engine.batch import StepEntry
from tokasaurus_amd.engine.runner import ModelRunner

MAX_LIVE = 4
ROUND_TO = 64


def parse_args(argv: list[str] | None = None) -> argparse.Namespace:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder the logits are written to")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    p.add_argument("--page-size", type=int, default=16, help="tokens per cache page (default 16)")
    return p.parse_args(argv)


def run(args: argparse.Namespace, lines=None, out=None) -> int:
    lines = lines if lines is not None else sys.stdin
    out = out if out is not None else sys.stdout
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    page = args.page_size
    if ROUND_TO % page and page % ROUND_TO:
        raise SystemExit(f"--page-size {page} neither divides {ROUND_TO} nor is a multiple of it")
    unit = max(page, ROUND_TO)
    tokens = -(-args.max_tokens // unit) * unit
    runner = ModelRunner.from_folder(
        args.model, args.dtype, page_size=page, num_pages=tokens // page, max_slots=MAX_LIVE
    )
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        entries = [StepEntry(str(e["id"]), [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
                   for e in rec.get("entries", [])]
        if entries:
            # a row's position: the tokens its request held before this step plus the wanted place
            held = {e.request_id: (runner.manager.requests[e.request_id].num_tokens
                                   if e.request_id in runner.manager.requests else 0) for e in entries}
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                np.ascontiguousarray(arr).tofile(out_dir / f"{rec['step']}.f32")
                rows = [[e.request_id, held[e.request_id] + w] for e in entries for w in e.want]
                (out_dir / f"{rec['step']}.json").write_text(
                    json.dumps({"step": rec["step"], "vocab": int(arr.shape[1]), "rows": rows}) + "\n")
        for rid in rec.get("end", []):
            # a request that never held anything (or was ended before) has nothing to give back
            if str(rid) in runner.manager.requests:
                runner.release(str(rid))
        print(f"done {rec['step']}", file=out, flush=True)
    return 0


def main(argv: list[str] | None = None) -> int:
    return run(parse_args(argv))
