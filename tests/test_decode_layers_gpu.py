"""The run of blocks in one kernel (an engine option, off by default): decode steps of few
requests through it give the plain model's logits in every cutting, agree with the separate
kernels, and a barrier across the grid that cannot complete ends in an error, not in a hang."""

import pytest
import torch

import plain_llama
from gpu_common import TOL, check_token_follows_plain
from replay_helpers import compare, mixed_trace, plain_rows, run_steps, tail_one_by_one
from tiny_models import TINY, random_tokens
from tokasaurus_amd import EngineConfig, SamplingParams
from tokasaurus_amd.engine.batch import StepEntry
from tokasaurus_amd.engine.engine import Engine
from tokasaurus_amd.engine.runner import ModelRunner
from tokasaurus_amd.kernels import ops
from tokasaurus_amd.kernels.library import KernelError

pytestmark = pytest.mark.gpu


def fused_runner(folders, name, tokens=512, **kw):
    _, page = TINY[name]
    runner = ModelRunner.from_folder(folders[name], "bfloat16", page_size=page, num_pages=tokens // page, max_slots=4, **kw)
    runner.model.fuse_decode = True
    return runner


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_decode_steps_through_the_one_kernel_run(folders, name):
    """Head sizes 16 to 64, pages of 4 to 32, groups of 2 and 3, widths that are no power of two:
    the last 32 tokens one by one (recorded steps of one row) and mixed batches on few pages
    (eager steps of up to four rows beside prompt portions, which take the separate kernels)."""
    cfg, _ = TINY[name]
    head_dim = cfg["hidden_size"] // cfg["num_attention_heads"]
    reqs = {f"r{n}": random_tokens(n, cfg["vocab_size"], 300 + n) for n in (70, 41, 97, 5)}
    ref = plain_rows(folders[name], reqs)
    runner = fused_runner(folders, name)
    before = ops.decode_layers_calls
    for rid in ("r70", "r97"):
        compare(run_steps(runner, tail_one_by_one(rid, reqs[rid], 32)), ref, **TOL["bfloat16"])
    got = run_steps(runner, mixed_trace(reqs, seed=9))
    assert len(got) == sum(len(t) for t in reqs.values())
    compare(got, ref, **TOL["bfloat16"])
    if head_dim in (16, 32, 64, 128):
        assert ops.decode_layers_calls > before, "no step went through the one-kernel run"
    else:
        assert ops.decode_layers_calls == before  # a head size it is not built for: the separate kernels ran
    assert runner.manager.num_free_pages() == [p.num_pages for p in runner.manager.pools]


def test_the_run_agrees_with_the_separate_kernels_and_the_engine_takes_the_option(folders):
    cfg, page = TINY["C"]
    prompts = [random_tokens(n, cfg["vocab_size"], 50 + n) for n in (9, 30, 17, 4, 22, 11)]
    params = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    done = {}
    for fused in (False, True):
        before = ops.decode_layers_calls
        engine = Engine(EngineConfig(model=str(folders["C"]), dtype="bfloat16", page_size=page, kv_cache_num_tokens=1024,
                                     max_seqs_per_forward=4, max_tokens_per_forward=64, fuse_decode_layers=fused))
        done[fused] = engine.generate(prompts, params)
        assert (ops.decode_layers_calls > before) == fused
    pcfg, w = plain_llama.load_folder(folders["C"])
    for prompt, c in zip(prompts, done[True]):
        ids = list(prompt)
        for tok in c.tokens:
            check_token_follows_plain(plain_llama.forward_logits(pcfg, w, ids)[-1], tok, 0.0, 0.0)
            ids.append(tok)
    # the two paths sum in different orders: the same tokens but for near ties, close log-probabilities
    for a, b in zip(done[False], done[True]):
        same = sum(x == y for x, y in zip(a.tokens, b.tokens))
        assert same >= len(a.tokens) - 2
        if a.tokens == b.tokens:
            assert torch.allclose(torch.tensor(a.logprobs), torch.tensor(b.logprobs), atol=0.08)


def test_a_barrier_that_cannot_complete_ends_in_an_error_and_the_next_step_works(folders):
    """The barrier is told to wait for one workgroup more than the grid has, with a spin limit
    of a few hundred polls: every workgroup gives up, runs to the end and exits (no access
    depends on what another workgroup should have written), the status word is set, and the
    host raises.  The barrier's memory is cleared then, and the same step runs again."""
    cfg, _ = TINY["C"]
    toks = random_tokens(40, cfg["vocab_size"], 3)
    ref = plain_rows(folders["C"], {"x": toks})
    runner = fused_runner(folders, "C", use_graphs=False)
    runner.step([StepEntry("x", toks[:39], [])])
    groups = ops.load("fused").tk_decode_layers_groups()
    real = ops.decode_layers

    def broken(*args, **kw):
        return real(*args, spin_cap=300, expect_groups=groups + 1, **kw)

    import tokasaurus_amd.models.causal_lm as causal_lm

    causal_lm.ops.decode_layers = broken
    try:
        with pytest.raises(KernelError, match="gave up waiting"):
            runner.step([StepEntry("x", [toks[39]], [0])])
    finally:
        causal_lm.ops.decode_layers = real
    # the failed step did not advance the request; the same token goes in again
    assert runner.manager.requests["x"].num_tokens == 39
    before = ops.decode_layers_calls
    logits = runner.step([StepEntry("x", [toks[39]], [0])])
    assert ops.decode_layers_calls == before + 1
    compare({("x", 39): logits[0].float().cpu()}, ref, **TOL["bfloat16"])
    runner.release("x")
