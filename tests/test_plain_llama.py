"""Pins the plain implementation by what fixes it beside the reference's text:
special cases that reduce to a library routine, and invariants chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, a wrong
head mapping, a mask off by one) fails one of them."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as pl
from tiny_models import CONFIG_A, CONFIG_B, make_folder, random_tokens

torch.manual_seed(0)


# ---- RMSNorm ---------------------------------------------------------------


def test_rms_norm_with_unit_weight_is_the_library_routine():
    x = torch.randn(5, 96)
    got = pl.rms_norm(x, torch.ones(96), 1e-6)
    assert torch.allclose(got, F.rms_norm(x, (96,), eps=1e-6), atol=1e-6)


def test_rms_norm_scale_invariance_and_row_norm():
    x = torch.randn(4, 64)
    a = pl.rms_norm(x, torch.ones(64), 1e-12)
    b = pl.rms_norm(7.5 * x, torch.ones(64), 1e-12)
    assert torch.allclose(a, b, atol=1e-5)
    assert torch.allclose(a.norm(dim=-1), torch.full((4,), math.sqrt(64)), atol=1e-3)


def test_rms_norm_casts_before_the_weight():
    # llama.py:51: weight * hidden.to(input_dtype): in bfloat16 the normalised value
    # is rounded first; multiplying in 32-bit and rounding once gives other bits.
    x = torch.randn(3, 64).bfloat16()
    w = (1 + 0.3 * torch.randn(64)).bfloat16()
    got = pl.rms_norm(x, w, 1e-5)
    xf = x.float()
    n = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)
    assert torch.equal(got, w * n.bfloat16())
    assert got.dtype == torch.bfloat16


# ---- linear ----------------------------------------------------------------


def test_linear_is_out_in_layout():
    x, w = torch.randn(3, 8), torch.randn(5, 8)
    assert torch.allclose(pl.linear(x, w), F.linear(x, w))


# ---- rotary ----------------------------------------------------------------


def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    d = 32
    inv = pl.rope_inverse_frequencies(d, 10000.0, None)
    x = torch.randn(6, 2, d)
    cos, sin = pl.rope_tables(torch.arange(6), inv)
    y = pl.apply_rope(x, cos, sin)
    assert torch.allclose(y[0], x[0], atol=1e-7)
    half = d // 2
    pair_norm = lambda t: t[..., :half] ** 2 + t[..., half:] ** 2  # lane j with lane j + d/2
    assert torch.allclose(pair_norm(y), pair_norm(x), atol=1e-5)
    assert torch.equal(cos[:, :half], cos[:, half:])
    assert cos.dtype == torch.float32


def test_rope_scores_depend_only_on_distance():
    d = 16
    inv = pl.rope_inverse_frequencies(d, 10000.0, None)
    q, k = torch.randn(1, 1, d), torch.randn(1, 1, d)

    def score(m, n):
        cq, sq = pl.rope_tables(torch.tensor([m]), inv)
        ck, sk = pl.rope_tables(torch.tensor([n]), inv)
        return (pl.apply_rope(q, cq, sq) * pl.apply_rope(k, ck, sk)).sum()

    assert torch.allclose(score(5, 2), score(40, 37), atol=1e-4)
    assert torch.allclose(score(9, 9), score(0, 0), atol=1e-4)
    assert not torch.allclose(score(5, 2), score(2, 5), atol=1e-3)  # the sign of the rotation matters


def test_rope_rotation_direction():
    # one pair (j=0, theta=1): position p rotates (1, 0) to (cos p, sin p)
    inv = torch.tensor([1.0])
    x = torch.tensor([[[1.0, 0.0]]])
    cos, sin = pl.rope_tables(torch.tensor([1]), inv)
    y = pl.apply_rope(x, cos, sin)[0, 0]
    assert torch.allclose(y, torch.tensor([math.cos(1.0), math.sin(1.0)]), atol=1e-6)


def test_llama3_scaling_bands():
    d, theta = 64, 500000.0
    base = pl.rope_inverse_frequencies(d, theta, None)
    same = pl.rope_inverse_frequencies(d, theta, dict(rope_type="llama3", factor=1.0, low_freq_factor=1.0,
                                                     high_freq_factor=4.0, original_max_position_embeddings=64))
    assert torch.allclose(base, same)
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    scaled = pl.rope_inverse_frequencies(d, theta, sc)
    wavelen = 2 * math.pi / base
    short, long_ = wavelen < 64 / 4.0, wavelen > 64 / 1.0
    assert short.any() and long_.any() and (~short & ~long_).any()
    assert torch.equal(scaled[short], base[short])  # high frequencies untouched
    assert torch.allclose(scaled[long_], base[long_] / 8.0)  # low frequencies divided by factor
    mid = scaled[~short & ~long_] / base[~short & ~long_]
    assert ((mid > 1 / 8.0) & (mid < 1.0)).all()
    assert (mid[1:] <= mid[:-1] + 1e-7).all()  # monotone across the band
    # linear scaling divides everything
    lin = pl.rope_inverse_frequencies(d, theta, dict(rope_type="linear", factor=4.0))
    assert torch.allclose(lin, base / 4.0)


@pytest.mark.parametrize("d, theta, factor, low, high, orig", [
    (32, 500000.0, 8.0, 1.0, 4.0, 64),      # tiny configuration B
    (64, 500000.0, 32.0, 1.0, 4.0, 8192),   # the 1B model's scaling
    (128, 500000.0, 8.0, 1.0, 4.0, 8192),   # the 8B model's
    (48, 10000.0, 4.0, 2.0, 8.0, 128),      # other factors: low_freq_factor is not 1
])
def test_llama3_blend_is_linear_in_frequency(d, theta, factor, low, high, orig):
    """The middle band by the definition itself, element by element in Python floats:
    s = (orig / wavelength - low) / (high - low) is linear in the FREQUENCY (not in the
    wavelength) and the result is (1 - s) * f / factor + s * f.  A blend linear in the
    wavelength, a blend of the angles' periods, or the two outer bands exchanged all fail this.
    The reference delegates the generator to an installed package, which this build neither
    reads nor imports: beyond this definition the parity of the blend is unpinned.  The
    engine's own generator (a separate implementation) must give the same numbers."""
    from tokasaurus_amd.parts.position import inverse_frequencies

    sc = dict(rope_type="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high,
              original_max_position_embeddings=orig)
    want, bands = [], set()
    for j in range(d // 2):
        f = theta ** (-2.0 * j / d)
        wavelength = 2.0 * math.pi / f
        if wavelength < orig / high:
            want.append(f)
            bands.add("short")
        elif wavelength > orig / low:
            want.append(f / factor)
            bands.add("long")
        else:
            s = (orig / wavelength - low) / (high - low)
            assert 0.0 <= s <= 1.0
            want.append((1.0 - s) * f / factor + s * f)
            bands.add("middle")
    assert bands == {"short", "long", "middle"}
    want = torch.tensor(want, dtype=torch.float64)
    for got in (pl.rope_inverse_frequencies(d, theta, sc), inverse_frequencies(d, theta, sc)):
        assert got.dtype == torch.float32
        assert torch.allclose(got.double(), want, rtol=2e-6, atol=0)
    # at the band's two edges the blend meets the outer bands: s = 0 where the wavelength is
    # orig / low and s = 1 where it is orig / high
    for edge, s_want in ((orig / low, 0.0), (orig / high, 1.0)):
        assert abs((orig / edge - low) / (high - low) - s_want) < 1e-12


# ---- attention -------------------------------------------------------------


def test_attention_is_the_library_routine_on_a_whole_sequence():
    T, nq, nkv, d = 11, 6, 2, 16
    q, k, v = torch.randn(T, nq, d), torch.randn(T, nkv, d), torch.randn(T, nkv, d)
    got = pl.causal_attention(q, k, v)
    kk = k.repeat_interleave(nq // nkv, dim=1)  # query head h reads kv head h // group
    vv = v.repeat_interleave(nq // nkv, dim=1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
    assert torch.allclose(got, ref.transpose(0, 1), atol=1e-5)


def test_attention_one_head_no_mask_needed_for_last_row():
    # the last query sees every key: plain softmax(q k^T / sqrt(d)) v
    T, d = 7, 8
    q, k, v = torch.randn(T, 1, d), torch.randn(T, 1, d), torch.randn(T, 1, d)
    got = pl.causal_attention(q, k, v)[-1, 0]
    p = torch.softmax(q[-1, 0] @ k[:, 0].T / math.sqrt(d), dim=-1)
    assert torch.allclose(got, p @ v[:, 0], atol=1e-6)
    assert torch.allclose(pl.causal_attention(q, k, v)[0, 0], v[0, 0], atol=1e-6)  # first row sees itself only


def test_attention_window():
    T, d, w = 9, 8, 3
    q, k, v = torch.randn(T, 1, d), torch.randn(T, 1, d), torch.randn(T, 1, d)
    got = pl.causal_attention(q, k, v, window=w)
    for t in (0, 2, 3, 8):
        lo = max(0, t - w + 1)
        ref = pl.causal_attention(q[lo : t + 1], k[lo : t + 1], v[lo : t + 1])[-1]
        assert torch.allclose(got[t], ref, atol=1e-6)


# ---- feed-forward, head, model ----------------------------------------------


def _tiny_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = H // nq
    w = {"model.embed_tokens.weight": torch.randn(V, H, generator=g) * 0.5,
         "model.norm.weight": 1 + 0.1 * torch.randn(H, generator=g)}
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = torch.randn(V, H, generator=g) * 0.1
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        w[f"{p}.input_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g)
        w[f"{p}.post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g)
        w[f"{p}.self_attn.q_proj.weight"] = torch.randn(nq * d, H, generator=g) * 0.2
        w[f"{p}.self_attn.k_proj.weight"] = torch.randn(nkv * d, H, generator=g) * 0.2
        w[f"{p}.self_attn.v_proj.weight"] = torch.randn(nkv * d, H, generator=g) * 0.1
        w[f"{p}.self_attn.o_proj.weight"] = torch.randn(H, nq * d, generator=g) * 0.1
        w[f"{p}.mlp.gate_proj.weight"] = torch.randn(I, H, generator=g) * 0.1
        w[f"{p}.mlp.up_proj.weight"] = torch.randn(I, H, generator=g) * 0.1
        w[f"{p}.mlp.down_proj.weight"] = torch.randn(H, I, generator=g) * 0.1
    return w


def test_swiglu_is_silu_times_up_and_zero_gate_gives_the_input_back():
    cfg = dict(CONFIG_A)
    w = _tiny_weights(cfg)
    x = torch.randn(4, cfg["hidden_size"])
    p = "model.layers.0"
    h = pl.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    ref = x + F.linear(F.silu(F.linear(h, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(h, w[f"{p}.mlp.up_proj.weight"]),
                       w[f"{p}.mlp.down_proj.weight"])
    assert torch.allclose(pl.swiglu_block(x, w, p, cfg), ref, atol=1e-5)
    w0 = dict(w)
    w0[f"{p}.mlp.gate_proj.weight"] = torch.zeros_like(w[f"{p}.mlp.gate_proj.weight"])
    assert torch.allclose(pl.swiglu_block(x, w0, p, cfg), x)


def test_head_tied_and_untied():
    for cfg in (CONFIG_A, CONFIG_B):
        w = _tiny_weights(cfg)
        x = torch.randn(2, cfg["hidden_size"])
        h = pl.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
        mat = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
        got = pl.lm_head(x, w, cfg)
        assert got.dtype == torch.float32
        assert torch.allclose(got, h @ mat.T, atol=1e-5)


@pytest.mark.parametrize("cfg", [CONFIG_A, CONFIG_B])
def test_model_is_causal_and_shift_invariant(cfg):
    w = _tiny_weights(cfg)
    toks = random_tokens(20, cfg["vocab_size"], 3)
    full = pl.forward_logits(cfg, w, toks)
    # causality: a prefix's logits do not change when tokens follow
    assert torch.allclose(pl.forward_logits(cfg, w, toks[:9]), full[:9], atol=1e-5)
    # only distances count: shifting every position leaves the logits unchanged.  With
    # llama3 scaling this still holds (scaling changes frequencies, not the relative form).
    shifted = pl.forward_logits(cfg, w, toks, first_position=37)
    assert torch.allclose(shifted, full, atol=2e-4)
    # but positions matter: swapping two prompt tokens changes later logits
    sw = list(toks)
    sw[2], sw[5] = sw[5], sw[2]
    assert not torch.allclose(pl.forward_logits(cfg, w, sw)[-1], full[-1], atol=1e-4)


def test_single_layer_model_by_hand():
    # one layer, one head, no grouping: the whole model written out with library calls
    cfg = dict(CONFIG_A, num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1)
    w = _tiny_weights(cfg)
    toks = random_tokens(6, cfg["vocab_size"], 5)
    H, eps = cfg["hidden_size"], cfg["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][toks]
    p = "model.layers.0"
    h = F.rms_norm(x, (H,), eps=eps) * w[f"{p}.input_layernorm.weight"]
    q, k, v = (F.linear(h, w[f"{p}.self_attn.{n}_proj.weight"]) for n in "qkv")
    inv = 1.0 / (cfg["rope_theta"] ** (torch.arange(0, H, 2).float() / H))
    ang = torch.arange(6).float()[:, None] * inv[None]
    c, s = torch.cat([ang.cos()] * 2, -1), torch.cat([ang.sin()] * 2, -1)
    rot = lambda t: t * c + torch.cat([-t[:, H // 2 :], t[:, : H // 2]], -1) * s
    a = F.scaled_dot_product_attention(rot(q)[None], rot(k)[None], v[None], is_causal=True)[0]
    x = x + F.linear(a, w[f"{p}.self_attn.o_proj.weight"])
    h = F.rms_norm(x, (H,), eps=eps) * w[f"{p}.post_attention_layernorm.weight"]
    x = x + F.linear(F.silu(F.linear(h, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(h, w[f"{p}.mlp.up_proj.weight"]),
                     w[f"{p}.mlp.down_proj.weight"])
    ref = F.linear(F.rms_norm(x, (H,), eps=eps) * w["model.norm.weight"], w["model.embed_tokens.weight"])
    assert torch.allclose(pl.forward_logits(cfg, w, toks), ref, atol=1e-4)


def test_layer_order_and_folder_loading(tmp_path):
    folder = make_folder(tmp_path / "a", CONFIG_A, seed=3)
    cfg, w = pl.load_folder(folder)
    assert all(t.dtype == torch.float32 for t in w.values())
    toks = random_tokens(12, cfg["vocab_size"], 1)
    assert torch.equal(pl.forward_logits(cfg, w, toks), pl.forward_logits(cfg, w, toks, layer_order=[0, 1]))
    assert not torch.allclose(pl.forward_logits(cfg, w, toks, layer_order=[1, 0]), pl.forward_logits(cfg, w, toks))


# ---- sampling --------------------------------------------------------------


def test_topk_logprobs():
    logits = torch.tensor([0.1, 2.0, -1.0, 3.0, 0.5])
    ids, lps = pl.topk_logprobs(logits, 0.5, 3)
    assert ids == [3, 1, 4]
    want = torch.log_softmax(logits / 0.5, -1)
    assert torch.allclose(torch.tensor(lps), want[[3, 1, 4]], atol=1e-6)
    # the first place is the greedy token with the log-probability the sampler reports for it
    tok, lp = pl.sample(logits, 0.0, 0.0)
    ids, lps = pl.topk_logprobs(logits, 0.0, 1)
    assert ids == [tok] and abs(lps[0] - lp) < 1e-6
    # all of them: the probabilities sum to one
    _, lps = pl.topk_logprobs(logits, 1.3, 5)
    assert abs(sum(math.exp(x) for x in lps) - 1.0) < 1e-5


def test_sampling():
    logits = torch.tensor([0.1, 2.0, -1.0, 2.0, 0.5])
    tok, lp = pl.sample(logits, 0.0, 0.3)
    assert tok == 1  # argmax of the raw logits, lowest index on a tie
    assert abs(lp - float(torch.log_softmax(logits, -1)[1])) < 1e-6
    probs = torch.softmax(logits / 0.7, -1)
    cdf = torch.cumsum(probs, -1)
    for u in (0.0, 0.05, 0.3, 0.6, 0.95, 0.999):
        tok, lp = pl.sample(logits, 0.7, u)
        assert tok == int((cdf > u).nonzero()[0])
        assert abs(lp - float(torch.log(probs[tok]))) < 1e-6
    # a small temperature agrees with greedy
    assert pl.sample(torch.tensor([0.1, 2.0, -1.0, 1.9]), 1e-3, 0.7)[0] == 1
    # frequencies over many uniforms match the probabilities
    us = torch.linspace(0, 1, 2001)[:-1]
    counts = torch.zeros(5)
    for u in us:
        counts[pl.sample(logits, 0.7, float(u))[0]] += 1
    assert torch.allclose(counts / len(us), probs, atol=2e-3)
