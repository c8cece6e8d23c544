"""The sampler's entry point that allocates nothing (tk_sample_static), called through ctypes
as a caller without torch's wrappers would: its tokens and log-probabilities equal those of
tk_sample with a caller's workspace, on two calls in a row, the second with a smaller input
(the static scratch then still holds what the first call left)."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

P = ctypes.c_void_p


def library():
    from tokasaurus_amd.kernels import build

    lib = ctypes.CDLL(str(build.ensure_built("core")))
    lib.tk_last_error.restype = ctypes.c_char_p
    lib.tk_sample_chunks.argtypes = [ctypes.c_int]
    lib.tk_sample_chunks.restype = ctypes.c_int
    lib.tk_sample.argtypes = [P, ctypes.c_int, ctypes.c_int, ctypes.c_int] + [P] * 10
    lib.tk_sample.restype = ctypes.c_int
    lib.tk_sample_static.argtypes = [P, ctypes.c_int, ctypes.c_int, ctypes.c_int] + [P] * 7
    lib.tk_sample_static.restype = ctypes.c_int
    return lib


def ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def case(rows, vocab, seed, slots_total):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn((rows, vocab), generator=g) * 3).cuda()
    temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.25 * (r % 4) for r in range(rows)], dtype=torch.float32).cuda()
    uniform = torch.rand((rows,), generator=g).cuda()
    slots = torch.randperm(slots_total, generator=g)[:rows].to(torch.int32).cuda()
    return logits, temperature, uniform, slots


def sample_both(lib, rows, vocab, seed):
    slots_total = 64
    logits, temperature, uniform, slots = case(rows, vocab, seed, slots_total)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    chunks = lib.tk_sample_chunks(vocab)
    out = {}
    for kind in ("workspace", "static"):
        ids = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        logprobs = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
        last_token = torch.full((slots_total,), -7, dtype=torch.int32, device="cuda")
        if kind == "workspace":
            part = torch.empty((3, rows * chunks), dtype=torch.float32, device="cuda")
            torch.cuda.synchronize()
            rc = lib.tk_sample(ptr(logits), logits.stride(0), rows, vocab, ptr(temperature), ptr(uniform), ptr(slots),
                               ptr(last_token), ptr(ids), ptr(logprobs), ptr(part[0]), ptr(part[1]), ptr(part[2]), stream)
        else:
            torch.cuda.synchronize()
            before = torch.cuda.memory_allocated()
            rc = lib.tk_sample_static(ptr(logits), logits.stride(0), rows, vocab, ptr(temperature), ptr(uniform),
                                      ptr(slots), ptr(last_token), ptr(ids), ptr(logprobs), stream)
            assert torch.cuda.memory_allocated() == before
        assert rc == 0, lib.tk_last_error().decode()
        torch.cuda.synchronize()
        out[kind] = (ids.cpu(), logprobs.cpu(), last_token.cpu())
    return out


def test_static_sampler_equals_the_one_with_a_workspace():
    lib = library()
    # the second call is smaller in rows and in vocabulary: stale partial results of the first
    # call lie in the scratch beside and behind what the second writes
    for rows, vocab, seed in ((48, 70001, 1), (5, 3001, 2), (1, 130, 3)):
        out = sample_both(lib, rows, vocab, seed)
        ids_w, lp_w, last_w = out["workspace"]
        ids_s, lp_s, last_s = out["static"]
        assert (ids_w >= 0).all() and (ids_w < vocab).all()
        assert torch.equal(ids_w, ids_s), (rows, vocab)
        assert torch.equal(lp_w, lp_s), (rows, vocab)  # the same kernels on the same numbers: the same bits
        assert torch.equal(last_w, last_s), (rows, vocab)


def test_static_sampler_refuses_what_its_scratch_cannot_hold():
    lib = library()
    vocab = 128256
    chunks = lib.tk_sample_chunks(vocab)
    rows = 16384 // chunks + 1
    logits, temperature, uniform, slots = case(2, vocab, 4, 8)
    ids = torch.zeros((rows,), dtype=torch.int32, device="cuda")
    # refused before anything is launched, so the short operands are never read
    rc = lib.tk_sample_static(ptr(logits), vocab, rows, vocab, ptr(temperature), ptr(uniform), None, None, ptr(ids), None,
                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc != 0
    assert "static scratch holds" in lib.tk_last_error().decode()
