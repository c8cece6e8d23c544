"""A causal language model built from a ``ModelSpec``: embedding, the blocks in
run order, final norm and head (the skeleton of tokasaurus/model/llama.py:521-582,
603-667 with the architecture taken out of it)."""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.models.spec import ModelSpec
from tokasaurus_amd.parts.base import (BLOCKS, EMBEDDINGS, HEADS, CacheNeed, CacheView, Part, Prepared, StateNeed, StepContext,
                                       TensorSpec)
from tokasaurus_amd.parts.block import build_with_shared, stream_and_prepared
import tokasaurus_amd.parts.embedding  # noqa: F401  (registers the embedding and the head)
from tokasaurus_amd.parts.linear import Placer


class CausalLM:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.shared: dict = {}
        self.embedding = build_with_shared(EMBEDDINGS, spec.embedding, self.shared)
        self.blocks = [build_with_shared(BLOCKS, b, self.shared) for b in spec.layers]
        self.head = build_with_shared(HEADS, spec.head, self.shared)
        self.dtype: torch.dtype | None = None
        self.device: torch.device | None = None
        self.weight_bytes = 0
        # True: decode steps of few tokens run neighbouring blocks that allow it in one kernel
        # (kernels.ops.decode_layers, experimental); False: every block launches its own kernels
        self.fuse_decode = False
        self._decode_runs: dict = {}

    # ---- tensors
    def parts(self) -> list[Part]:
        return [self.embedding, *self.blocks, self.head]

    def tensor_specs(self) -> list[TensorSpec]:
        seen: dict[str, TensorSpec] = {}
        for part in self.parts():
            for s in part.tensor_specs():
                if s.name in seen and seen[s.name].shape != s.shape:
                    raise ValueError(f"tensor {s.name} is wanted with shapes {seen[s.name].shape} and {s.shape}")
                seen.setdefault(s.name, s)
        return list(seen.values())

    def load(self, tensors: dict[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        placer = Placer(dtype, device)
        for part in self.parts():
            part.load(tensors, placer)
        self.dtype, self.device = dtype, device
        self.weight_bytes = placer.bytes_placed()

    # ---- what the cache manager must provide, one item per run entry
    def cache_needs(self) -> list[CacheNeed | None]:
        return [self.blocks[e.layer].mixer.cache_need() for e in self.spec.run_order]

    def state_needs(self) -> list[StateNeed | None]:
        return [self.blocks[e.layer].mixer.state_need() for e in self.spec.run_order]

    # ---- one step
    def forward(
        self,
        ctx: StepContext,
        caches: list[CacheView | None],
        states: list[torch.Tensor | None],
        want_rows: torch.Tensor | None,
    ) -> torch.Tensor:
        """Run the batch of ``ctx`` and return logits [len(want_rows), vocab] in 32-bit;
        ``want_rows`` None stands for every row in order (no rows are picked out then)."""
        x = self.embedding.forward(ctx)
        order = self.spec.run_order
        last = len(order) - 1
        prepared = None  # what a block has done for the norm that the next one (or the head) starts with
        runs = self._decode_runs_for(ctx, caches, states, want_rows)
        i = -1
        while i < last:
            i += 1
            entry = order[i]
            if i in runs:
                # blocks i .. end - 1 in one kernel; it leaves what the norm behind the run needs
                end, run = runs[i]
                next_norm = self.blocks[order[end].layer].entry_norm() if end <= last else self.head.entry_norm()
                emit = next_norm.weight if getattr(next_norm, "fusable_rms", False) else None
                x, data = ops.decode_layers(run, x, ctx.positions, ctx.kv_len, [caches[j].block_table for j in range(i, end)],
                                            int(ctx.extras.get("kv_bound", 0)) or ctx.max_kv_len, emit_weight=emit)
                prepared = Prepared(data, next_norm) if data is not None else None
                ctx.extras["decode_layers"] = True
                i = end - 1
                continue
            rows = want_rows if i == last else None
            block = self.blocks[entry.layer]
            if block.fuses_norm:
                next_norm = self.blocks[order[i + 1].layer].entry_norm() if i < last else self.head.entry_norm()
                out = block.forward(x, ctx, caches[i], states[i], rows, prepared=prepared, next_norm=next_norm)
            else:
                out = block.forward(x, ctx, caches[i], states[i], rows)
            x, prepared = stream_and_prepared(out)
        if last < 0 and want_rows is not None:
            x = ops.gather_rows(x, want_rows)
        return self.head.forward(x, prepared)

    def _decode_runs_for(self, ctx: StepContext, caches, states, want_rows) -> dict:
        """Runs of neighbouring run entries that one kernel can execute in this step, by their
        first entry: {first: (end, ops.DecodeLayers)}.  Only for steps of one token a request
        and few of them, in bfloat16, where every row goes on to the head; a run's blocks all
        offer their share (``Block.decode_fusion``) and have the same sizes."""
        if (not self.fuse_decode or ctx.max_q_len != 1 or not 0 < ctx.num_tokens <= ops.DECODE_LAYERS_ROWS
                or ctx.num_requests != ctx.num_tokens or self.dtype != torch.bfloat16 or want_rows is not None):
            return {}
        order = self.spec.run_order
        specs = []
        for i, entry in enumerate(order):
            spec = self.blocks[entry.layer].decode_fusion(caches[i], states[i])
            specs.append(spec)
        runs: dict = {}
        i = 0
        while i < len(order):
            if specs[i] is None:
                i += 1
                continue
            end = i + 1
            while end < len(order) and specs[end] is not None and specs[end].shape_key() == specs[i].shape_key():
                end += 1
            page_size = caches[i].page_size
            # the descriptors in device memory are made once per run and set of pages
            key = (i, end, page_size, tuple(s.kcache.data_ptr() for s in specs[i:end]))
            run = self._decode_runs.get(key)
            if run is None:
                run = ops.DecodeLayers(specs[i:end], page_size)
                self._decode_runs[key] = run
            # the tables change from step to step: the run's table numbers follow their order of first use
            if run.supports(ctx.num_tokens) and self._tables_match(run, specs[i:end]):
                runs[i] = (end, run)
            i = end
        return runs

    @staticmethod
    def _tables_match(run, specs) -> bool:
        """This step's block tables group the run's blocks as they did when the run was set up."""
        seen: list[int] = []
        for s, idx in zip(specs, run.table_of):
            key = id(s.block_table)
            if key not in seen:
                seen.append(key)
            if seen.index(key) != idx:
                return False
        return True
