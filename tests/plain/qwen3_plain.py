"""Plain Qwen3 forward: one function per part, whole sequences, no cache, CPU torch.

Every function cites the lines of the reference's source files whose formula it
restates.  Inputs are ordinary tensors and numbers; there is no module tree, no
batching trick and no key/value cache, so a mistake in the engine's cache or batch
handling cannot be mirrored here.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------- files


def read_model_dir(model_dir, dtype=torch.float32):
    """Read config.json and every tensor of every *.safetensors file in a folder.

    Mirrors engine/models/_loader.py:64-76 (all files, all keys, to CPU).  Tensors
    are upcast to `dtype` so the plain forward runs in one precision.
    """
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    tensors = {}
    for file in sorted(model_dir.glob("*.safetensors")):
        with safe_open(str(file), framework="pt", device="cpu") as f:
            for key in f.keys():
                t = f.get_tensor(key)
                tensors[key] = t.to(dtype) if t.is_floating_point() else t
    return cfg, tensors


# --------------------------------------------------------------------------- parts


def rms_norm(x, weight, eps):
    """y = x * rsqrt(mean(x^2, -1) + eps) * w, all in float32.

    engine/kernels/triton/rmsnorm.py:19-42 (the op Qwen3-0.6B runs: sum of squares,
    rstd = rsqrt(sum/DIM + eps), x*rstd*w with one rounding at the store);
    engine/nn/base_layers.py:39-46 is the same formula with an earlier cast.
    """
    xf = x.float()
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * rstd * weight.float()).to(x.dtype)


def rope_inv_freq(head_dim, theta):
    """inv_freq[i] = 1 / theta^(2i/head_dim), i = 0..head_dim/2-1, float32.

    engine/nn/rope.py:28-29.
    """
    idx = torch.arange(0, head_dim, 2, dtype=torch.float32)
    return 1.0 / (theta ** (idx / head_dim))


def rope_cos_sin(positions, head_dim, theta):
    """cos/sin of angle = float32(pos) * inv_freq, each [T, head_dim/2], float32.

    engine/nn/rope.py:105-109 (outer(positions, inv_freq) in float32, then cos, sin);
    engine/kernels/triton/rope.py:33-34,50-51 forms the same float32 product.
    """
    angles = torch.outer(positions.to(torch.float32), rope_inv_freq(head_dim, theta))
    return angles.cos(), angles.sin()


def apply_rope(x, cos, sin):
    """Rotate-half pairing (x[i], x[i+hd/2]) on x [T, heads, hd].

    out[i]       = x[i]      * cos - x[i+hd/2] * sin
    out[i+hd/2]  = x[i+hd/2] * cos + x[i]      * sin
    engine/kernels/triton/rope.py:53-65; engine/nn/rope.py:113-123 (x*cos +
    rotate_half(x)*sin with rotate_half = cat(-x2, x1)) is the same map.
    """
    half = x.shape[-1] // 2
    xf = x.float()
    re, im = xf[..., :half], xf[..., half:]
    c, s = cos[:, None, :], sin[:, None, :]
    out = torch.cat((re * c - im * s, im * c + re * s), dim=-1)
    return out.to(x.dtype)


def causal_attention(q, k, v, window=None):
    """Causal softmax attention of one whole sequence with grouped query heads.

    q [T, nq, hd], k/v [T, nkv, hd].  Query head j reads key/value head
    j // (nq // nkv); scores are scaled by hd^-0.5; the token at position p sees
    keys 0..p (engine/nn/sdpa.py:56,85-102: softmax_scale=hd^-0.5, causal=True,
    window_size=(-1,-1), softcap 0).  `window` = W keeps only keys p-W+1..p; the
    reference never sets one (engine/models/_registry.py:20 is unread), so that
    branch has no counterpart there.
    """
    T, nq, hd = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    qf, kf, vf = q.float(), k.float(), v.float()
    pos = torch.arange(T)
    visible = pos[None, :] <= pos[:, None]
    if window is not None:
        visible &= pos[None, :] > pos[:, None] - window
    out = torch.empty(T, nq, hd, dtype=torch.float32)
    for j in range(nq):
        kj, vj = kf[:, j // group], vf[:, j // group]
        scores = (qf[:, j] @ kj.T) * (hd ** -0.5)
        scores = scores.masked_fill(~visible, float("-inf"))
        out[:, j] = torch.softmax(scores, dim=-1) @ vj
    return out.to(q.dtype)


def attention_mixer(h, w, prefix, positions, *, num_heads, num_kv_heads, head_dim,
                    eps, theta, window=None):
    """q/k/v projections, per-head RMSNorm on q and k, RoPE, attention, o projection.

    engine/nn/attention.py:171-198: projections (no bias for Qwen3), unflatten to
    heads, q_norm/k_norm over head_dim with one weight vector shared by all heads
    (:178-182) BEFORE the rotation (:184), v untouched, attention, flatten, o_proj.
    """
    T = h.shape[0]
    q = h @ w[prefix + "q_proj.weight"].T
    k = h @ w[prefix + "k_proj.weight"].T
    v = h @ w[prefix + "v_proj.weight"].T
    q = q.view(T, num_heads, head_dim)
    k = k.view(T, num_kv_heads, head_dim)
    v = v.view(T, num_kv_heads, head_dim)
    q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
    cos, sin = rope_cos_sin(positions, head_dim, theta)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    o = causal_attention(q, k, v, window=window)
    return o.reshape(T, num_heads * head_dim) @ w[prefix + "o_proj.weight"].T


def swiglu(h, w, prefix):
    """down(silu(gate(h)) * up(h)), no bias.  engine/nn/layers.py:65-66."""
    gate = h @ w[prefix + "gate_proj.weight"].T
    up = h @ w[prefix + "up_proj.weight"].T
    return (torch.nn.functional.silu(gate) * up) @ w[prefix + "down_proj.weight"].T


def layer_windows(cfg):
    """Per-layer window (None = all keys) from Qwen3's config.json keys.

    The reference has no windowed layers; this only reads the keys Qwen3's own
    config.json carries (`layer_types`, `sliding_window`, `use_sliding_window`,
    `max_window_layers`).
    """
    n = cfg["num_hidden_layers"]
    win = cfg.get("sliding_window")
    types = cfg.get("layer_types")
    if types is not None:
        return [win if t == "sliding_attention" else None for t in types]
    if cfg.get("use_sliding_window") and win is not None:
        first = cfg.get("max_window_layers", n)
        return [win if i >= first else None for i in range(n)]
    return [None] * n


def forward_hidden(cfg, w, token_ids, positions=None):
    """Embedding, every pre-norm block, final norm: hidden states [T, H].

    engine/model.py:58-73; block = engine/nn/layers.py:111-121
    (x = x + attn(attn_norm(x)); x = x + ffn(ffn_norm(x))).
    """
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    T = ids.shape[0]
    if positions is None:
        positions = torch.arange(T)
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nq)
    hd = cfg.get("head_dim", cfg["hidden_size"] // nq)
    eps = cfg["rms_norm_eps"]
    windows = layer_windows(cfg)
    x = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_mixer(
            h, w, p + "self_attn.", positions, num_heads=nq, num_kv_heads=nkv,
            head_dim=hd, eps=eps, theta=cfg["rope_theta"], window=windows[i])
        h = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(h, w, p + "mlp.")
    return rms_norm(x, w["model.norm.weight"], eps)


def lm_head(cfg, w, hidden):
    """Tied: x E^T (engine/nn/layers.py:22-23); untied: x Wlm^T, no bias
    (HF lm_head has none; engine/models/qwen/_checkpoint.py:23,51-62)."""
    if cfg.get("tie_word_embeddings", False):
        return hidden @ w["model.embed_tokens.weight"].T
    return hidden @ w["lm_head.weight"].T


def forward_logits(cfg, w, token_ids, positions=None):
    """Logits [T, V] at every position of one whole sequence."""
    return lm_head(cfg, w, forward_hidden(cfg, w, token_ids, positions)).float()


# --------------------------------------------------------------------------- sampling


def greedy_generate(cfg, w, prompt, max_tokens):
    """Argmax decoding by re-running the whole sequence for every new token."""
    ids = list(prompt)
    for _ in range(max_tokens):
        ids.append(int(forward_logits(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


def sampling_distribution(logits, temperature):
    """softmax(logits / T) in float32.  engine/generation/sampler.py:11-12."""
    return torch.softmax(logits.float() / temperature, dim=-1)


def sample_with_noise(logits, temperature, exponential_noise):
    """argmax(probs / max(noise, 1e-10)) with noise ~ Exp(1).

    engine/generation/sampler.py:13-15.
    """
    probs = sampling_distribution(logits, temperature)
    return int((probs / exponential_noise.clamp_min(1e-10)).argmax(dim=-1))
