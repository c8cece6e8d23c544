"""Plain 32-bit references of single kernels, for the per-kernel GPU tests.
They work on host tensors and share no code with the engine."""

from __future__ import annotations

import math

import torch


def pack_key_pages(k: torch.Tensor) -> torch.Tensor:
    """[pages, nkv, P, d] -> the engine's key pages [pages, nkv, d / 8, P, 8]."""
    pages, nkv, P, d = k.shape
    return k.reshape(pages, nkv, P, d // 8, 8).permute(0, 1, 3, 2, 4).contiguous()


def unpack_key_pages(k: torch.Tensor) -> torch.Tensor:
    pages, nkv, pieces, P, eight = k.shape
    return k.permute(0, 1, 3, 2, 4).reshape(pages, nkv, P, pieces * eight)


def pack_value_pages(v: torch.Tensor) -> torch.Tensor:
    """[pages, nkv, d, P] -> the engine's value pages [pages, nkv, P / 4, d, 4]."""
    pages, nkv, d, P = v.shape
    return v.reshape(pages, nkv, d, P // 4, 4).permute(0, 1, 3, 2, 4).contiguous()


def unpack_value_pages(v: torch.Tensor) -> torch.Tensor:
    pages, nkv, quads, d, four = v.shape
    return v.permute(0, 1, 3, 2, 4).reshape(pages, nkv, d, quads * four)


def make_paged_case(
    q_lens: list[int],
    kv_lens: list[int],
    nq: int,
    nkv: int,
    d: int,
    page: int,
    seed: int,
    dtype: torch.dtype,
    sharp: float = 3.0,
    spare_pages: int = 3,
    poison: bool = True,
):
    """A batch of requests with shuffled pages.  Returns host tensors:
    q [N, nq*d], dense keys/values per request, the paged caches
    (packed as the engine keeps them), block table, q_start, kv_len.
    Queries are scaled so that scores have a spread of about ``sharp``: a
    missing or misplaced key then moves the result far beyond rounding.
    Unused cache entries are NaN when ``poison`` (nothing stale may be read)."""
    g = torch.Generator().manual_seed(seed)
    R = len(q_lens)
    blocks = [-(-n // page) for n in kv_lens]
    total_pages = sum(blocks) + spare_pages
    perm = torch.randperm(total_pages, generator=g).tolist()
    width = max(blocks)
    table = torch.full((R, width), -1, dtype=torch.int32)
    fill = float("nan") if poison else 0.0
    kc = torch.full((total_pages, nkv, page, d), fill, dtype=torch.float32)
    vc = torch.full((total_pages, nkv, d, page), fill, dtype=torch.float32)
    dense_k, dense_v, qs = [], [], []
    at = 0
    for r in range(R):
        k = torch.randn((kv_lens[r], nkv, d), generator=g).to(dtype).float()
        v = torch.randn((kv_lens[r], nkv, d), generator=g).to(dtype).float()
        q = (torch.randn((q_lens[r], nq, d), generator=g) * sharp).to(dtype).float()
        dense_k.append(k)
        dense_v.append(v)
        qs.append(q.reshape(q_lens[r], nq * d))
        for b in range(blocks[r]):
            p = perm[at]
            at += 1
            table[r, b] = p
            n = min(page, kv_lens[r] - b * page)
            kc[p, :, :n, :] = k[b * page : b * page + n].permute(1, 0, 2)
            vc[p, :, :, :n] = v[b * page : b * page + n].permute(1, 2, 0)
    q_start = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    return {
        "q": torch.cat(qs, 0),
        "k": dense_k,
        "v": dense_v,
        "kcache": pack_key_pages(kc),
        "vcache": pack_value_pages(vc),
        "table": table,
        "q_start": q_start,
        "kv_len": torch.tensor(kv_lens, dtype=torch.int32),
    }


def attention_reference(case, q_lens, kv_lens, nq, nkv, d, window: int = 0, scale: float | None = None) -> torch.Tensor:
    """Per request and head: softmax(q k^T * scale) v over positions lo..pos of each
    token (bottom-right aligned causal mask), in 64-bit."""
    scale = scale if scale is not None else 1.0 / math.sqrt(d)
    group = nq // nkv
    outs = []
    at = 0
    for r, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        q = case["q"][at : at + ql].view(ql, nq, d).double()
        at += ql
        k, v = case["k"][r].double(), case["v"][r].double()
        out = torch.empty((ql, nq, d), dtype=torch.float64)
        pos = torch.arange(kl - ql, kl)
        keys = torch.arange(kl)
        allowed = keys[None, :] <= pos[:, None]
        if window > 0:
            allowed &= keys[None, :] > pos[:, None] - window
        for h in range(nq):
            s = (q[:, h] @ k[:, h // group].T) * scale
            s = s.masked_fill(~allowed, float("-inf"))
            out[:, h] = torch.softmax(s, -1) @ v[:, h // group]
        outs.append(out.reshape(ql, nq * d))
    return torch.cat(outs, 0).float()
