"""The step function: one batch of (request, its next tokens) through the model.

``ModelRunner`` owns the model, the cache manager and the cache tensors.  A step
runs only the tokens it is given, as one batch, reading everything earlier from
the cache, and returns the logits at the wanted places in 32-bit.  It is the
counterpart of the reference's preprocess/run_model pair
(tokasaurus/model/basic_worker.py:57-139) without the sampling, which sits on
top (the reference's forward never returns logits, tokasaurus/model/types.py:403-425).
"""

from __future__ import annotations

from pathlib import Path

import torch

from tokasaurus_amd.cache.manager import CacheManager, plan_groups
from tokasaurus_amd.cache.storage import CacheStorage
from tokasaurus_amd.engine.batch import PlannedEntry, StepEntry, layout, to_device
from tokasaurus_amd.models.causal_lm import CausalLM
from tokasaurus_amd.models.registry import build_model, config_from_folder
from tokasaurus_amd.parts.base import CacheView
from tokasaurus_amd.weights.loader import read_tensors

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: this engine has no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


class ModelRunner:
    def __init__(
        self,
        model: CausalLM,
        page_size: int,
        num_pages: int,
        max_slots: int,
    ):
        assert model.device is not None, "load the model's weights first"
        self.model = model
        self.page_size = page_size
        self.max_positions = model.spec.max_positions
        needs = model.cache_needs()
        cache_of = [e.cache_of for e in model.spec.run_order]
        self.groups, self.where = plan_groups(needs, cache_of)
        self.manager = CacheManager(self.groups, num_pages, page_size, max_slots)
        self.storage = CacheStorage(
            self.groups,
            [num_pages] * len(self.groups),
            page_size,
            model.state_needs(),
            max_slots,
            model.dtype,
            model.device,
        )

    # ---- construction from a model folder
    @classmethod
    def from_folder(
        cls,
        model_dir: str | Path,
        dtype: str,
        page_size: int,
        num_pages: int,
        max_slots: int,
        rope_scaling_override: tuple[bool, dict | None] = (False, None),
    ) -> "ModelRunner":
        device = require_gpu()
        if dtype not in DTYPES:
            raise ValueError(f"dtype {dtype!r}: this engine runs {sorted(DTYPES)}")
        arch, cfg = config_from_folder(model_dir, rope_scaling_override)
        model = build_model(arch, cfg)
        specs = model.tensor_specs()
        # a checkpoint that ties its head may still carry the head's tensor
        allow = ("lm_head.weight",) if model.spec.head_name == model.spec.embedding_name else ()
        tensors = read_tensors(model_dir, specs, allow_unexpected=allow)
        model.load(tensors, DTYPES[dtype], device)
        return cls(model, page_size, num_pages, max_slots)

    # ---- requests
    def admit(self, request_id: str) -> None:
        self.manager.admit(request_id)

    def release(self, request_id: str) -> None:
        self.manager.release(request_id)

    # ---- the step
    def plan(self, entries: list[StepEntry]) -> list[PlannedEntry]:
        """Reserve pages for every entry (NoSpaceException leaves the cache usable)."""
        planned = []
        for e in entries:
            if e.request_id not in self.manager.requests:
                self.manager.admit(e.request_id)
            rc = self.manager.requests[e.request_id]
            q_len = 1 if e.tokens is None else len(e.tokens)
            new_len = rc.num_tokens + q_len
            if new_len > self.max_positions:
                raise ValueError(
                    f"request {e.request_id!r} would reach {new_len} tokens, the model's positions end at {self.max_positions}"
                )
            self.manager.reserve(e.request_id, new_len)
            planned.append(PlannedEntry(e.request_id, e.tokens, list(e.want), rc.slot, rc.num_tokens, rc.tables))
        return planned

    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Run one batch; logits [wanted, vocab] float32 in the order of the
        entries and of their ``want`` lists."""
        planned = self.plan(entries)
        hb = layout(planned, self.model.spec.vocab_size, len(self.groups))
        ctx, want_rows, tables = to_device(hb, self.model.dtype, self.model.device, self.storage.last_token)
        caches: list[CacheView | None] = []
        for i, w in enumerate(self.where):
            if w is None:
                caches.append(None)
                continue
            g, k = w
            caches.append(
                CacheView(
                    keys=self.storage.keys[g][k],
                    values=self.storage.values[g][k],
                    block_table=tables[g],
                    page_size=self.page_size,
                    writable=self.model.spec.run_order[i].cache_of is None,
                )
            )
        logits = self.model.forward(ctx, caches, self.storage.states, want_rows)
        for e in planned:
            self.manager.advance(e.request_id, e.start + e.q_len)
        return logits
