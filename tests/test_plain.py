"""What fixes the plain implementation beside the reference's text: special cases that
reduce to a library routine, invariants, and the shapes the reference's own tests use.
Each check is chosen so that a plausible misreading (a wrong sign or pairing, a norm in
the wrong place, a wrong head grouping) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from helpers import TINY_A, TINY_B, TINY_C, random_prompt
from plain import qwen3_plain as plain
from tokensprint_amd.weights import random_tensors


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("shape", [(257, 1024), (4, 73, 1024)])   # the reference's shapes
def test_rms_norm_is_the_library_routine(shape):
    x = rnd(*shape)
    w = torch.rand(shape[-1], generator=torch.Generator().manual_seed(1)) * 2 - 1
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-6), F.rms_norm(x, shape[-1:], w, 1e-6),
                               rtol=1e-5, atol=1e-6)


def test_rms_norm_invariants():
    x = rnd(5, 64)
    ones = torch.ones(64)
    y = plain.rms_norm(x, ones, 1e-6)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(5), rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(plain.rms_norm(7.0 * x, ones, 1e-12), plain.rms_norm(x, ones, 1e-12),
                               rtol=1e-5, atol=1e-6)            # scale invariance as eps -> 0
    # eps is inside the root: a zero row stays zero, not NaN
    assert torch.equal(plain.rms_norm(torch.zeros(1, 8), torch.ones(8), 1e-6), torch.zeros(1, 8))


# ------------------------------------------------------------------ rotation
def test_rope_frequencies():
    # engine/nn/rope.py:28-29; the reference's tests/test_rope_scaling.py:63-79
    f = plain.rope_inv_freq(8, 10000.0)
    assert f[0] == 1.0
    torch.testing.assert_close(f, torch.tensor([10000.0 ** (-2 * i / 8) for i in range(4)]))


def test_rope_position_zero_is_identity_and_norms_are_kept():
    x = rnd(6, 3, 16)
    cos, sin = plain.rope_cos_sin(torch.zeros(6, dtype=torch.long), 16, 1e6)
    torch.testing.assert_close(plain.apply_rope(x, cos, sin), x)
    cos, sin = plain.rope_cos_sin(torch.arange(6) * 37, 16, 1e4)
    y = plain.apply_rope(x, cos, sin)
    pair = lambda t: t[..., :8] ** 2 + t[..., 8:] ** 2      # pairs are (i, i + hd/2)
    torch.testing.assert_close(pair(y), pair(x), rtol=1e-5, atol=1e-6)
    # interleaved pairing (2i, 2i+1) would not keep these pair norms
    wrong = lambda t: t[..., 0::2] ** 2 + t[..., 1::2] ** 2
    assert not torch.allclose(wrong(y), wrong(x), rtol=1e-3, atol=1e-3)


def test_rope_scores_depend_on_distance_only_and_sign_is_right():
    q, k = rnd(1, 1, 16, seed=1), rnd(1, 1, 16, seed=2)

    def score(p, s):
        cq, sq = plain.rope_cos_sin(torch.tensor([p]), 16, 100.0)
        ck, sk = plain.rope_cos_sin(torch.tensor([s]), 16, 100.0)
        return (plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum()

    torch.testing.assert_close(score(9, 4), score(25, 20), rtol=1e-4, atol=1e-5)
    assert not torch.allclose(score(9, 4), score(4, 9), rtol=1e-3, atol=1e-4)
    # a unit vector on the first pair turns counter-clockwise by pos * inv_freq[0] = pos
    e = torch.zeros(1, 1, 16); e[0, 0, 0] = 1.0
    c, s = plain.rope_cos_sin(torch.tensor([1]), 16, 100.0)
    y = plain.apply_rope(e, c, s)
    torch.testing.assert_close(y[0, 0, 0], torch.tensor(math.cos(1.0)))
    torch.testing.assert_close(y[0, 0, 8], torch.tensor(math.sin(1.0)))


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("nq,nkv", [(4, 4), (8, 2), (6, 3), (1, 1)])
def test_attention_is_the_library_routine(nq, nkv):
    T, hd = 23, 16
    q, k, v = rnd(T, nq, hd, seed=1), rnd(T, nkv, hd, seed=2), rnd(T, nkv, hd, seed=3)
    ref = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
        is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    torch.testing.assert_close(plain.causal_attention(q, k, v), ref, rtol=1e-5, atol=1e-5)


def test_attention_first_token_and_window():
    T, hd = 12, 8
    q, k, v = rnd(T, 2, hd, seed=1), rnd(T, 1, hd, seed=2), rnd(T, 1, hd, seed=3)
    out = plain.causal_attention(q, k, v)
    torch.testing.assert_close(out[0, 0], v[0, 0])            # one key: its value
    torch.testing.assert_close(plain.causal_attention(q, k, v, window=1)[:, 1], v[:, 0])
    torch.testing.assert_close(plain.causal_attention(q, k, v, window=T), out)
    w3 = plain.causal_attention(q, k, v, window=3)
    for p in (5, 11):
        part = plain.causal_attention(q[p - 2:p + 1], k[p - 2:p + 1], v[p - 2:p + 1])
        torch.testing.assert_close(w3[p], part[-1], rtol=1e-5, atol=1e-6)


def test_head_grouping_is_by_blocks():
    # query head j reads key/value head j // group: heads 0,1 -> 0 and 2,3 -> 1
    T, hd = 5, 8
    q = rnd(T, 4, hd)
    k = rnd(T, 2, hd, seed=1)
    v = torch.zeros(T, 2, hd); v[:, 0] = 1.0; v[:, 1] = -1.0
    out = plain.causal_attention(q, k, v)
    torch.testing.assert_close(out[:, :2], torch.ones(T, 2, hd))
    torch.testing.assert_close(out[:, 2:], -torch.ones(T, 2, hd))


# ------------------------------------------------------------------ feed-forward, block
def test_swiglu():
    h = rnd(7, 12)
    w = {"gate_proj.weight": rnd(20, 12, seed=1), "up_proj.weight": rnd(20, 12, seed=2),
         "down_proj.weight": rnd(12, 20, seed=3)}
    ref = (F.silu(h @ w["gate_proj.weight"].T) * (h @ w["up_proj.weight"].T)) @ w["down_proj.weight"].T
    torch.testing.assert_close(plain.swiglu(h, w, ""), ref)
    w["gate_proj.weight"] = torch.zeros(20, 12)
    assert plain.swiglu(h, w, "").abs().max() == 0


def weights(cfg, seed):
    return random_tensors(cfg, seed, torch.float32)


def test_block_is_identity_when_output_projections_are_zero():
    w = weights(TINY_B, 1)
    for i in range(3):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    ids = random_prompt(9, 389, 0)
    hidden = plain.forward_hidden(TINY_B, w, ids)
    ref = plain.rms_norm(w["model.embed_tokens.weight"][ids], w["model.norm.weight"], 1e-5)
    torch.testing.assert_close(hidden, ref)


def test_qk_norm_comes_before_the_rotation_and_v_is_untouched():
    # with unit norm weights every q/k head vector entering the rotation has RMS 1, so
    # scaling the q projection by 10 cannot change the output; scaling v must scale it
    w = weights(TINY_A, 0)
    ids = random_prompt(8, 256, 1)
    pos = torch.arange(8)
    h = rnd(8, 64)
    kw = dict(num_heads=4, num_kv_heads=2, head_dim=16, eps=1e-9, theta=1e4)
    p = "model.layers.0.self_attn."
    base = plain.attention_mixer(h, w, p, pos, **kw)
    w2 = dict(w); w2[p + "q_proj.weight"] = 10 * w[p + "q_proj.weight"]
    torch.testing.assert_close(plain.attention_mixer(h, w2, p, pos, **kw), base, rtol=1e-4, atol=1e-6)
    w3 = dict(w); w3[p + "v_proj.weight"] = 10 * w[p + "v_proj.weight"]
    torch.testing.assert_close(plain.attention_mixer(h, w3, p, pos, **kw), 10 * base, rtol=1e-4, atol=1e-6)


def test_logits_depend_on_distances_only():
    # shifting all positions by a constant changes no score, hence no logit
    w = weights(TINY_A, 0)
    ids = random_prompt(10, 256, 2)
    a = plain.forward_logits(TINY_A, w, ids)
    b = plain.forward_logits(TINY_A, w, ids, positions=torch.arange(10) + 40)
    torch.testing.assert_close(a, b, rtol=1e-3, atol=1e-4)


def test_causality_and_the_head():
    w = weights(TINY_B, 1)
    ids = random_prompt(12, 389, 3)
    full = plain.forward_logits(TINY_B, w, ids)
    torch.testing.assert_close(plain.forward_logits(TINY_B, w, ids[:7]), full[:7], rtol=1e-4, atol=1e-5)
    hidden = plain.forward_hidden(TINY_B, w, ids)
    torch.testing.assert_close(full, F.linear(hidden, w["lm_head.weight"]))      # untied
    wa = weights(TINY_A, 0)
    ids_a = random_prompt(5, 256, 5)
    ha = plain.forward_hidden(TINY_A, wa, ids_a)
    torch.testing.assert_close(plain.forward_logits(TINY_A, wa, ids_a),
                               F.linear(ha, wa["model.embed_tokens.weight"]))   # tied


def test_windowed_layers_differ_from_full_ones_only_beyond_the_window():
    w = weights(TINY_C, 2)
    ids = random_prompt(60, 301, 4)
    full_cfg = {**TINY_C, "layer_types": ["full_attention"] * 4}
    a, b = plain.forward_logits(TINY_C, w, ids), plain.forward_logits(full_cfg, w, ids)
    torch.testing.assert_close(a[:24], b[:24])          # window 24: first 24 positions agree
    assert not torch.allclose(a[40:], b[40:], rtol=1e-3, atol=1e-4)


# ------------------------------------------------------------------ sampling
def test_sampler_formulas():
    logits = rnd(50)
    p = plain.sampling_distribution(logits, 0.7)
    torch.testing.assert_close(p.sum(), torch.tensor(1.0))
    assert plain.sample_with_noise(logits, 1e-4, torch.ones(50)) == int(logits.argmax())
    g = torch.Generator().manual_seed(0)
    draws = torch.tensor([plain.sample_with_noise(logits[:6], 0.7,
                                                  torch.empty(6).exponential_(1, generator=g))
                          for _ in range(6000)])
    freq = torch.bincount(draws, minlength=6).float() / 6000
    assert (freq - plain.sampling_distribution(logits[:6], 0.7)).abs().max() < 0.03
