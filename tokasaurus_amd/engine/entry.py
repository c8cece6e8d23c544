"""The command line, in the reference's manner: ``toka key=value ...``
(tokasaurus/entry.py:139-143, README.md:93-146).  The reference's command starts
a server; this engine has none, so the command generates completions for token
ids given on the command line, or for seeded random prompts, and prints one
JSON object per completion and a final line of statistics.

    toka model=DIR prompt_ids='([[1, 2, 3]])' max_tokens=8
    toka model=DIR random_weights=T seed=3 num_prompts=4 prompt_len=100 temperature=0.8
    toka model=DIR dtype=float32 kv_cache_num_tokens='(64*1024)' .eager
"""

from __future__ import annotations

import json
import sys
from contextlib import contextmanager
from dataclasses import dataclass
from pathlib import Path

from tokasaurus_amd.config.engine_config import EngineConfig, OptionError, apply_overrides


@dataclass
class RunConfig(EngineConfig):
    """The engine's options plus what the command itself needs."""

    random_weights: bool = False  # write model.safetensors into `model` from its config.json and `seed`
    prompt_ids: list | None = None  # one prompt [ids] or several [[ids], ...]
    num_prompts: int = 1  # without prompt_ids: seeded random prompts
    prompt_len: int = 32
    max_tokens: int = 16
    temperature: float = 0.0
    ignore_eos: bool = False
    topk_logprobs: int | None = None  # per token, this many most probable tokens (needs max_topk_logprobs)


def prepare_model_folder(config: RunConfig) -> None:
    if config.model is None:
        raise OptionError("model=DIR is required")
    folder = Path(config.model)
    if config.random_weights and not (folder / "model.safetensors").exists():
        from tokasaurus_amd.weights import write_random_model

        cfg_path = folder / "config.json"
        if not cfg_path.is_file():
            raise OptionError(f"random_weights=T needs {cfg_path} to say which model to make")
        write_random_model(folder, json.loads(cfg_path.read_text()), config.seed)
        print(f"wrote random weights (seed {config.seed}) to {folder}", file=sys.stderr)
    elif not folder.is_dir():
        raise OptionError(f"model folder {folder} does not exist (only local folders are read)")


@contextmanager
def engine_manager(config: EngineConfig):
    """``with engine_manager(config) as engine:`` — the counterpart of the
    reference's ``server_manager`` (tokasaurus/entry.py:90-111), yielding the
    in-process engine instead of starting server processes."""
    from tokasaurus_amd.engine.engine import Engine

    engine = Engine(config)
    try:
        yield engine
    finally:
        del engine


def start(config: RunConfig) -> int:
    import torch

    from tokasaurus_amd.engine.engine import Engine
    from tokasaurus_amd.sampling import SamplingParams

    prepare_model_folder(config)
    engine = Engine(config)
    vocab = engine.runner.model.spec.vocab_size
    if config.prompt_ids is not None:
        prompts = config.prompt_ids
        if prompts and not isinstance(prompts[0], list):
            prompts = [prompts]
    else:
        g = torch.Generator().manual_seed(config.seed)
        prompts = [torch.randint(0, vocab, (config.prompt_len,), generator=g).tolist() for _ in range(config.num_prompts)]
    params = SamplingParams(temperature=config.temperature, max_tokens=config.max_tokens, ignore_eos=config.ignore_eos,
                            topk_logprobs=config.topk_logprobs)
    for c in engine.generate(prompts, params):
        line = {"id": c.request_id, "tokens": c.tokens, "logprobs": c.logprobs, "finish_reason": c.finish_reason}
        if c.topk_ids is not None:
            line["topk_ids"], line["topk_logprobs"] = c.topk_ids, c.topk_logprobs
        print(json.dumps(line))
    print(json.dumps({"stats": engine.stats.as_dict()}), file=sys.stderr)
    return 0


def main(argv: list[str] | None = None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    try:
        config = apply_overrides(RunConfig(), argv)
        return start(config)
    except ValueError as e:  # an option, or a request the engine refuses: say so without a traceback
        print(f"toka: {e}", file=sys.stderr)
        return 2


if __name__ == "__main__":
    sys.exit(main())
