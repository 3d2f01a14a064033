"""Tiny configurations and small helpers shared by the tests."""

from __future__ import annotations

import torch


def qwen3_config(*, hidden, layers, heads, kv_heads, head_dim, inter, vocab, eps, theta,
                 tied, max_pos, window=None, layer_types=None):
    cfg = {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
        "hidden_size": hidden, "num_hidden_layers": layers, "num_attention_heads": heads,
        "num_key_value_heads": kv_heads, "head_dim": head_dim, "intermediate_size": inter,
        "vocab_size": vocab, "rms_norm_eps": eps, "rope_theta": theta,
        "max_position_embeddings": max_pos, "tie_word_embeddings": tied,
        "hidden_act": "silu", "attention_bias": False, "rope_scaling": None,
        "sliding_window": window, "use_sliding_window": window is not None,
    }
    if layer_types is not None:
        cfg["layer_types"] = layer_types
    return cfg


# Two configurations that differ in every size and option, plus one with windowed
# layers.  A and B are the two tiny configurations the benchmark description names.
TINY_A = qwen3_config(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=16, inter=128,
                      vocab=256, eps=1e-6, theta=10000.0, tied=True, max_pos=128)
TINY_B = qwen3_config(hidden=96, layers=3, heads=8, kv_heads=2, head_dim=32, inter=160,
                      vocab=389, eps=1e-5, theta=1e6, tied=False, max_pos=256)
TINY_C = qwen3_config(hidden=80, layers=4, heads=6, kv_heads=3, head_dim=48, inter=112,
                      vocab=301, eps=3e-6, theta=50000.0, tied=False, max_pos=512,
                      window=24, layer_types=["full_attention", "sliding_attention",
                                              "sliding_attention", "full_attention"])
# head size 64: the smallest one the decode-fused kernels take
TINY_D = qwen3_config(hidden=128, layers=2, heads=4, kv_heads=1, head_dim=64, inter=200,
                      vocab=515, eps=2e-6, theta=2e5, tied=True, max_pos=320)
TINY = {"A": (TINY_A, 0, 4), "B": (TINY_B, 1, 16), "C": (TINY_C, 2, 8),
        "D": (TINY_D, 3, 32)}   # cfg, seed, page


# Two layers of the Qwen3-0.6B shape with a vocabulary wide enough for the output head's
# own kernels: the widths at which the K-splitting products, their fused norm forms and
# the fused decode attention serve an engine (the tiny widths above take other kernels).
# GPU tests only.
LAYER_E = qwen3_config(hidden=1024, layers=2, heads=16, kv_heads=8, head_dim=128, inter=3072,
                       vocab=20011, eps=1e-6, theta=1e6, tied=True, max_pos=256)
# Two layers of the Qwen3-8B and Qwen3-32B shapes: at these widths other routes serve the
# rows (the library from 16 rows on, the norm as a kernel of its own where the fused form's
# limits end, key/value groups of 4 and 8 query heads).
LAYER_F = qwen3_config(hidden=4096, layers=2, heads=32, kv_heads=8, head_dim=128, inter=12288,
                       vocab=20011, eps=1e-6, theta=1e6, tied=False, max_pos=256)
LAYER_G = qwen3_config(hidden=5120, layers=2, heads=64, kv_heads=8, head_dim=128, inter=25600,
                       vocab=20011, eps=1e-6, theta=1e6, tied=False, max_pos=256)
GPU_ONLY = {"E": (LAYER_E, 4, 16), "F": (LAYER_F, 5, 16), "G": (LAYER_G, 6, 16)}
# The same widths with a windowed layer beside a full one: two cache groups, so that a
# step (a captured decode step too) carries two block tables and the window's kernels run
# at the widths of real models.
WINDOWED = {name + "W": (dict(cfg, sliding_window=40, use_sliding_window=True,
                              layer_types=["sliding_attention", "full_attention"]), seed + 10, page)
            for name, (cfg, seed, page) in GPU_ONLY.items()}


def random_prompt(length, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


def write_word_tokenizer(model_dir, vocab_size, *, eos_id=2, name_eos=True, pad_id=None):
    """A word-level tokenizer for `vocab_size` ids in `model_dir`, as checkpoint folders
    hold one: tokenizer.json (word i is "w<i>", split at white space; id 0 is the unknown
    word, `eos_id` the end-of-sequence token, both special) and tokenizer_config.json."""
    import json
    from pathlib import Path

    from tokenizers import Tokenizer, models, pre_tokenizers

    words = {f"w{i}": i for i in range(vocab_size)}
    words = {("<unk>" if i == 0 else "<eos>" if i == eos_id else "<pad>" if i == pad_id else w): i
             for w, i in words.items()}
    tok = Tokenizer(models.WordLevel(words, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.add_special_tokens(["<unk>", "<eos>"] + (["<pad>"] if pad_id is not None else []))
    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    tok.save(str(model_dir / "tokenizer.json"))
    named = {"unk_token": "<unk>"}
    if name_eos:
        named["eos_token"] = {"content": "<eos>", "special": True}
    if pad_id is not None:
        named["pad_token"] = "<pad>"
    (model_dir / "tokenizer_config.json").write_text(json.dumps(named))
    return tok
