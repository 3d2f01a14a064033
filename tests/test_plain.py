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
    # engine/nn/rope.py:28-29; the reference's tests/test_rope_scaling.py:63-79 pins the same
    # base frequencies.  By hand for head size 8 and base 10^4: 10^(-i), i = 0..3
    torch.testing.assert_close(plain.rope_inv_freq(8, 10000.0),
                               torch.tensor([1.0, 0.1, 0.01, 0.001]))
    f = plain.rope_inv_freq(128, 1e6)
    assert f.shape == (64,) and f[0] == 1.0 and f.dtype == torch.float32
    # a geometric sequence that ends one step short of 1/base
    torch.testing.assert_close(f[1:] / f[:-1], torch.full((63,), 1e6 ** (-1 / 64)))
    torch.testing.assert_close(f[-1] * 1e6 ** (-1 / 64), torch.tensor(1e-6))


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


def test_rope_is_a_complex_multiplication():
    # The rotate-half form of engine/kernels/triton/rope.py:53-65 and engine/nn/rope.py:
    # element i and element i + hd/2 are the real and imaginary part of one complex
    # number, multiplied by exp(i * pos * inv_freq[i]).  Written with the library's complex
    # arithmetic, which knows nothing of halves, signs or tables; the interleaved pairing
    # (2i, 2i+1) and the conjugate rotation both fail it.
    hd, theta = 32, 1e4
    x = rnd(7, 3, hd, seed=5)
    pos = torch.tensor([0, 1, 2, 17, 100, 211, 300])     # (float32 angles: pos * 6e-8 of error)
    cos, sin = plain.rope_cos_sin(pos, hd, theta)
    got = plain.apply_rope(x, cos, sin)
    z = torch.complex(x[..., :hd // 2].double(), x[..., hd // 2:].double())
    freq = theta ** (-torch.arange(0, hd, 2, dtype=torch.float64) / hd)
    turn = torch.polar(torch.ones(7, hd // 2, dtype=torch.float64), pos[:, None].double() * freq)
    want = z * turn[:, None, :]
    torch.testing.assert_close(got[..., :hd // 2].double(), want.real, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(got[..., hd // 2:].double(), want.imag, rtol=1e-4, atol=1e-4)
    other = z * turn.conj()[:, None, :]
    assert (got[..., hd // 2:].double() - other.imag).abs().max() > 0.1
    zi = torch.view_as_complex(x.double().reshape(7, 3, hd // 2, 2).contiguous()) * turn[:, None, :]
    interleaved = torch.view_as_real(zi).reshape(7, 3, hd)
    assert (got.double() - interleaved).abs().max() > 0.1


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


def _mixer_by_hand(h, w, p, pos, *, norm_first, eps, theta=1e4, nq=4, nkv=2, hd=16):
    """The attention mixer put together here from the pinned pieces, with the per-head norm
    before the rotation (`norm_first`) or after it."""
    T = h.shape[0]
    q = (h @ w[p + "q_proj.weight"].T).view(T, nq, hd)
    k = (h @ w[p + "k_proj.weight"].T).view(T, nkv, hd)
    v = (h @ w[p + "v_proj.weight"].T).view(T, nkv, hd)
    cos, sin = plain.rope_cos_sin(pos, hd, theta)
    norm = lambda t, name: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w[p + name]
    if norm_first:
        q, k = norm(q, "q_norm.weight"), norm(k, "k_norm.weight")
    q, k = plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin)
    if not norm_first:
        q, k = norm(q, "q_norm.weight"), norm(k, "k_norm.weight")
    o = plain.causal_attention(q, k, v)
    return o.reshape(T, nq * hd) @ w[p + "o_proj.weight"].T


def test_qk_norm_comes_before_the_rotation_and_v_is_untouched():
    # engine/nn/attention.py:178-184.  The rotation keeps a head vector's length, so only
    # the norm's weight tells the two orders apart: it must differ between the two
    # elements of a rotated pair.  Both orders are computed here; the plain mixer must be
    # the first and must not be the second.
    w = weights(TINY_A, 0)
    p = "model.layers.0.self_attn."
    w[p + "q_norm.weight"] = torch.linspace(0.3, 2.5, 16)
    w[p + "k_norm.weight"] = torch.linspace(1.9, 0.4, 16)
    pos = torch.arange(8) * 5 + 3
    h = 4 * rnd(8, 64)
    kw = dict(num_heads=4, num_kv_heads=2, head_dim=16, eps=1e-6, theta=1e4)
    got = plain.attention_mixer(h, w, p, pos, **kw)
    before = _mixer_by_hand(h, w, p, pos, norm_first=True, eps=1e-6)
    after = _mixer_by_hand(h, w, p, pos, norm_first=False, eps=1e-6)
    torch.testing.assert_close(got, before, rtol=1e-5, atol=1e-6)
    assert (got - after).abs().max() > 100 * (got - before).abs().max() + 1e-3
    # v is neither normed nor rotated: scaling its projection scales the output
    w3 = dict(w); w3[p + "v_proj.weight"] = 10 * w[p + "v_proj.weight"]
    torch.testing.assert_close(plain.attention_mixer(h, w3, p, pos, **kw), 10 * got,
                               rtol=1e-4, atol=1e-6)


def test_qk_norm_uses_the_given_eps():
    # the per-head norms take the same eps as the block norms (config.json has one
    # rms_norm_eps; the reference's separate qk_norm_eps has the same value,
    # engine/models/qwen/_archs.py:103,122).  With head vectors whose mean square is near
    # eps, the value of eps shows in the output.
    w = weights(TINY_A, 0)
    p = "model.layers.0.self_attn."
    pos = torch.arange(8)
    h = 0.02 * rnd(8, 64)                      # q, k elements of about 3e-3: mean square 1e-5
    kw = dict(num_heads=4, num_kv_heads=2, head_dim=16, theta=1e4)
    got = plain.attention_mixer(h, w, p, pos, eps=1e-5, **kw)
    torch.testing.assert_close(got, _mixer_by_hand(h, w, p, pos, norm_first=True, eps=1e-5),
                               rtol=1e-5, atol=1e-9)
    other = _mixer_by_hand(h, w, p, pos, norm_first=True, eps=1e-6)
    assert (got - other).abs().max() > 1e-2 * got.abs().max()
    # and the model passes config.json's rms_norm_eps down to them
    ids = random_prompt(9, 256, 1)
    small = dict(w)
    for i in range(2):
        for name in ("q_proj", "k_proj"):
            key = f"model.layers.{i}.self_attn.{name}.weight"
            small[key] = 0.01 * w[key]
    a = plain.forward_logits({**TINY_A, "rms_norm_eps": 1e-6}, small, ids)
    b = plain.forward_logits({**TINY_A, "rms_norm_eps": 1e-5}, small, ids)
    c = plain.forward_logits({**TINY_A, "rms_norm_eps": 1e-5}, w, ids)
    d = plain.forward_logits({**TINY_A, "rms_norm_eps": 1e-6}, w, ids)
    assert (a - b).abs().max() > 10 * (c - d).abs().max()


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
