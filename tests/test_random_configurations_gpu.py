"""Configurations drawn at random (head sizes in steps of 16 up to 128, odd numbers of heads
and groups, widths and vocabularies that are no power of two, one to three layers, with and
without rotary scaling, pages of 4 to 64) replayed in mixed batches on few pages, in 32-bit and
in bfloat16, against the plain implementation."""

import random

import pytest
import torch

import plain_llama
from gpu_common import TOL
from replay_helpers import compare, compare_with_bfloat16_measure, mixed_trace, plain_rows, run_steps
from tiny_models import make_folder, random_tokens
from tokasaurus_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu


def random_config(rng: random.Random) -> dict:
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 2, 3, 5, 8])
    group = rng.choice([1, 2, 3, 4, 5, 7, 8])
    while nkv * group * d > 3072:  # wider sums outgrow the 32-bit bound of the tiny models
        if group > 1:
            group -= 1
        else:
            nkv = max(1, nkv // 2)
    scaling = None
    if rng.random() < 0.6:
        scaling = {"rope_type": "llama3", "factor": rng.choice([2.0, 8.0, 32.0]), "low_freq_factor": 1.0,
                   "high_freq_factor": rng.choice([2.0, 4.0]),
                   "original_max_position_embeddings": rng.choice([32, 64, 128])}
    return {
        "architectures": ["LlamaForCausalLM"],
        "model_type": "llama",
        "num_hidden_layers": rng.choice([1, 2, 3]),
        "hidden_size": nkv * group * d,
        "num_attention_heads": nkv * group,
        "num_key_value_heads": nkv,
        "intermediate_size": rng.choice([8 * rng.randint(10, 60), rng.randint(80, 500)]),
        "vocab_size": rng.randint(100, 3000),
        "rope_theta": rng.choice([10000.0, 500000.0, 777.0]),
        "rope_scaling": scaling,
        "rms_norm_eps": rng.choice([1e-5, 1e-6, 1e-3]),
        "tie_word_embeddings": rng.random() < 0.5,
        "max_position_embeddings": 1024,
    }


@pytest.mark.parametrize("seed", [0, 1, 5, 9, 17, 23, 31, 40])
def test_a_random_configuration_in_mixed_batches(tmp_path, seed):
    rng = random.Random(seed)
    cfg = random_config(rng)
    page = rng.choice([4, 8, 16, 32, 64])
    folder = make_folder(tmp_path / "m", cfg, seed=seed)
    lengths = [rng.randint(1, 200) for _ in range(rng.randint(3, 7))]
    print(f"seed {seed}: page {page}, lengths {lengths}, {cfg}")
    requests = {f"r{i}": random_tokens(n, cfg["vocab_size"], 1000 * seed + i) for i, n in enumerate(lengths)}
    plain = plain_rows(folder, requests)
    cfg16, w16 = plain_llama.load_folder(folder, torch.bfloat16)
    plain16 = {rid: plain_llama.forward_logits(cfg16, w16, toks) for rid, toks in requests.items()}
    tokens = sum(sorted(-(-n // 64) * 64 for n in lengths)[-4:])  # room for the four longest only
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner.from_folder(folder, dtype, page_size=page, num_pages=-(-tokens // page), max_slots=4)
        got = run_steps(runner, mixed_trace(requests, seed=seed))
        assert len(got) == sum(lengths)
        if dtype == "float32":
            compare(got, plain, **TOL[dtype])
        else:
            compare_with_bfloat16_measure(got, plain, plain16, **TOL[dtype])
        assert runner.manager.num_free_pages() == [p.num_pages for p in runner.manager.pools]
