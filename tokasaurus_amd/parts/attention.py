"""Grouped-query attention over the paged cache
(tokasaurus/model/llama.py:96-287, tokasaurus/model/attention_utils.py:87-175).

q, k and v are one stacked product; the rotation of q and k is fused with the
append of k and v to the request's pages; one attention call then serves
prompt portions and single decoded tokens alike, each token reading the keys
at positions up to its own (bottom-right aligned causal mask), optionally only
the last ``window`` of them.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import (
    MIXERS,
    POSITION_ENCODINGS,
    CacheNeed,
    CacheView,
    Mixer,
    Normed,
    PartSpec,
    StepContext,
    TensorSpec,
)
from tokasaurus_amd.parts.linear import Linear, Placer


@dataclass
class AttentionPlan:
    """How the step's rows are cut into tiles and its keys into splits; made once
    a step for each group size and shared by the layers."""

    tile_req: torch.Tensor
    tile_row0: torch.Tensor
    row_tiles: int
    max_kv_len: int
    split: int
    waves: int
    scratch: ops.AttentionScratch | None = None  # a replayed step keeps its own


def attention_plan(ctx: StepContext, group: int, nkv: int) -> AttentionPlan:
    key = ("attention_plan", group, nkv)
    plan = ctx.extras.get(key)
    if plan is None:
        q_lens = [ctx.host_q_start[i + 1] - ctx.host_q_start[i] for i in range(ctx.num_requests)]
        row_tiles = 2 if ctx.max_q_len * group > 16 else 1
        tile_req, tile_row0 = ops.attention_tiles(q_lens, group, row_tiles)
        tiles = torch.tensor([tile_req, tile_row0], dtype=torch.int32).to(ctx.device)
        split, waves = ops.attention_split(ctx.max_kv_len, len(tile_req), nkv)
        plan = AttentionPlan(tiles[0], tiles[1], row_tiles, ctx.max_kv_len, split, waves)
        if ctx.extras.get("static"):
            plan.scratch = ops.AttentionScratch(ctx.device)
        ctx.extras[key] = plan
    return plan


@MIXERS.register("paged_attention")
class PagedAttention(Mixer):
    fuses_norm = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        names: dict[str, str],
        position: PartSpec | None = None,
        window: int = 0,
        shared: dict | None = None,
    ):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.window = int(window)
        self.scale = 1.0 / math.sqrt(head_dim)
        self.qkv = Linear(
            hidden_size,
            [names["q"], names["k"], names["v"]],
            [num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim],
        )
        self.out = Linear(num_heads * head_dim, [names["o"]], [hidden_size])
        self.position = None
        if position is not None:
            shared = shared if shared is not None else {}
            self.position = shared.setdefault(("position", position), POSITION_ENCODINGS.build(position))

    def tensor_specs(self) -> list[TensorSpec]:
        return self.qkv.tensor_specs() + self.out.tensor_specs()

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.num_kv_heads, self.head_dim, self.window)

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.qkv.load(tensors, placer)
        self.out.load(tensors, placer)
        if self.position is not None:
            self.position.prepare(placer.device)

    def forward(
        self,
        h: torch.Tensor | Normed,
        residual: torch.Tensor,
        ctx: StepContext,
        cache: CacheView | None,
        state: torch.Tensor | None,
        rows: torch.Tensor | None,
        emit_norm=None,
    ):
        assert cache is not None, "paged attention needs a cache"
        nq, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        cos = self.position.cos if self.position is not None else None
        sin = self.position.sin if self.position is not None else None
        q = None
        if cache.writable:
            # few rows in bfloat16: one kernel multiplies, rotates and appends
            q = self.qkv.rope_append(h, ops.RopeAppend(
                ctx.positions, ctx.token_req, cache.block_table, cos, sin, cache.keys, cache.values,
                nq, nkv, d, cache.page_size))
        if q is None:
            # an entry that reads another entry's cache computes only its queries
            q = self.qkv(h, rows=None if cache.writable else nq * d)
            ops.rope_append(
                q, ctx.positions, ctx.token_req, cache.block_table, cos, sin,
                cache.keys, cache.values, nq, nkv, d, cache.page_size, write_cache=cache.writable,
            )
        if ops.attention_mfma_supports(q.dtype, d, cache.page_size):
            plan = attention_plan(ctx, nq // nkv, nkv)
            attn = ops.paged_attention_mfma(
                q, cache.keys, cache.values, cache.block_table, ctx.q_start, ctx.kv_len,
                plan.tile_req, plan.tile_row0, plan.row_tiles, nq, nkv, d, cache.page_size,
                plan.max_kv_len, plan.split, window=self.window, scale=self.scale, waves=plan.waves, scratch=plan.scratch,
            )
        else:
            # the true 32-bit path, and shapes the matrix-core kernel does not take
            attn = ops.paged_attention_generic(
                q, cache.keys, cache.values, cache.block_table, ctx.token_req, ctx.positions,
                nq, nkv, d, cache.page_size, window=self.window, scale=self.scale,
            )
        if rows is not None:
            attn = ops.gather_rows(attn, rows)
        return self.out.with_residual(attn, residual, emit_norm)
