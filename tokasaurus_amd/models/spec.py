"""A model as data: which parts each layer is made of, and in which order the
layers run.

``run_order`` is a list of entries; an entry names a layer (the same layer may
be named twice: its weights are then used twice, each use with a cache of its
own) and may name an earlier entry whose cache it reads instead of keeping one.
"""

from __future__ import annotations

from dataclasses import dataclass

from tokasaurus_amd.parts.base import PartSpec


@dataclass(frozen=True)
class RunEntry:
    layer: int
    cache_of: int | None = None  # index into run_order of the entry whose cache is read


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    embedding: PartSpec  # chosen from parts.base.EMBEDDINGS
    head: PartSpec  # chosen from parts.base.HEADS (a head that names the embedding's tensor shares its buffer)
    layers: tuple[PartSpec, ...]  # block arrangements, each naming its own parts
    run_order: tuple[RunEntry, ...]
    max_positions: int
    eos_token_ids: tuple[int, ...] = ()
    # tensors a checkpoint of this architecture may carry although the model reads them from
    # elsewhere (the head's matrix of a checkpoint that ties it to the embedding)
    ignorable_tensors: tuple[str, ...] = ()

    def validate(self) -> None:
        for i, e in enumerate(self.run_order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run entry {i} names layer {e.layer}, the model has {len(self.layers)}")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"run entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if self.run_order[e.cache_of].cache_of is not None:
                    raise ValueError(f"run entry {i} reads the cache of entry {e.cache_of}, which keeps none itself")
