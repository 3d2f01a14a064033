"""Weights by name: dtype rules, one error for everything wrong, random-weights mode."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY_A, TINY_B
from kernel_refs import TorchOps
from tokensprint_amd.engine.assemble import build_model, load_model
from tokensprint_amd.parts.base import TensorDecl
from tokensprint_amd.weights import (WeightsError, declared_tensors, held_dtype, load_weights,
                                     random_tensors, write_random_model)


def test_declared_names_are_the_checkpoint_names():
    names = set(declared_tensors(TINY_B))
    assert "model.embed_tokens.weight" in names and "lm_head.weight" in names
    assert "model.norm.weight" in names
    for i in range(3):
        p = f"model.layers.{i}."
        for n in ("self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight",
                  "self_attn.o_proj.weight", "self_attn.q_norm.weight", "self_attn.k_norm.weight",
                  "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight",
                  "input_layernorm.weight", "post_attention_layernorm.weight"):
            assert p + n in names
    assert len(names) == 3 * 11 + 3
    d = declared_tensors(TINY_B)
    assert d["model.layers.0.self_attn.q_proj.weight"].shape == (8 * 32, 96)
    assert d["model.layers.0.self_attn.k_proj.weight"].shape == (2 * 32, 96)
    assert d["model.layers.0.self_attn.q_norm.weight"].shape == (32,)


def test_random_model_folder(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_A, seed=0, dtype=torch.bfloat16)
    cfg = json.loads((d / "config.json").read_text())
    assert cfg["hidden_size"] == 64 and cfg["torch_dtype"] == "bfloat16"
    t = load_file(str(d / "model.safetensors"))
    assert "lm_head.weight" not in t                      # tied: no separate head
    assert all(v.dtype == torch.bfloat16 for v in t.values())
    w = t["model.layers.0.mlp.up_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    n = t["model.norm.weight"].float()
    assert 0.89 < n.min() and n.max() < 1.11 and n.std() > 0.02
    # same seed, same tensors; another seed, others
    again = random_tensors(cfg, 0, torch.bfloat16)
    assert all(torch.equal(again[k], t[k]) for k in t)
    other = random_tensors(cfg, 1, torch.bfloat16)
    assert not torch.equal(other["model.norm.weight"], t["model.norm.weight"])


def test_held_dtypes():
    mat, vec, tab = TensorDecl((2, 2)), TensorDecl((2,), "vector"), TensorDecl((2,), "table")
    bf, f32 = torch.bfloat16, torch.float32
    assert held_dtype(mat, bf, bf) == bf and held_dtype(mat, torch.float16, bf) == bf
    assert held_dtype(mat, f32, bf) == f32          # stored in 32-bit: stays so
    assert held_dtype(mat, bf, f32) == f32
    assert held_dtype(vec, bf, bf) == f32           # small vectors: float32, exact
    assert held_dtype(tab, torch.int64, bf) == torch.int32


def _model(cfg, dtype="float32"):
    return build_model(cfg, dtype, "cpu", ops=TorchOps())[1]


def test_tied_head_shares_the_embedding(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_A, 0, torch.float32)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    assert model.head.weight.data_ptr() == model.embedding.table.data_ptr()
    # a tied file that still carries lm_head.weight loads, and the copy is ignored
    t = load_file(str(d / "model.safetensors"))
    t["lm_head.weight"] = torch.zeros_like(t["model.embed_tokens.weight"])
    save_file(t, str(d / "model.safetensors"))
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    assert model.head.weight.data_ptr() == model.embedding.table.data_ptr()


def test_bf16_run_keeps_32bit_tensors(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_B, 1, torch.bfloat16)
    t = load_file(str(d / "model.safetensors"))
    t["model.layers.1.mlp.down_proj.weight"] = t["model.layers.1.mlp.down_proj.weight"].float()
    save_file(t, str(d / "model.safetensors"))
    _, model = load_model(d, "bfloat16", "cpu", ops=TorchOps())
    assert model.blocks[1].feed_forward.w_down.dtype == torch.float32
    assert model.blocks[0].feed_forward.w_down.dtype == torch.bfloat16
    assert model.blocks[0].mixer_norm.weight.dtype == torch.float32


def test_bf16_run_warns_about_32bit_matrices_and_can_round_them(tmp_path, caplog):
    d = write_random_model(tmp_path / "m", TINY_B, 1, torch.float32)
    with caplog.at_level("WARNING"):
        _, model = load_model(d, "bfloat16", "cpu", ops=TorchOps())
    assert model.blocks[0].feed_forward.w_down.dtype == torch.float32
    assert "stay so in this bfloat16 run" in caplog.text and "cast_32bit=True" in caplog.text
    caplog.clear()
    with caplog.at_level("WARNING"):
        _, model = load_model(d, "bfloat16", "cpu", ops=TorchOps(), cast_32bit=True)
    assert not caplog.text
    assert model.blocks[0].feed_forward.w_down.dtype == torch.bfloat16
    assert model.embedding.table.dtype == torch.bfloat16
    assert model.blocks[0].mixer_norm.weight.dtype == torch.float32       # vectors stay float32
    ref = load_file(str(d / "model.safetensors"))["model.layers.0.mlp.down_proj.weight"]
    assert torch.equal(model.blocks[0].feed_forward.w_down, ref.to(torch.bfloat16))
    # a float32 run holds everything in float32 whatever is asked
    _, model = load_model(d, "float32", "cpu", ops=TorchOps(), cast_32bit=True)
    assert model.blocks[0].feed_forward.w_down.dtype == torch.float32


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_B, 1, torch.float32)
    t = load_file(str(d / "model.safetensors"))
    del t["model.layers.2.self_attn.k_norm.weight"], t["lm_head.weight"]
    t["model.layers.0.mlp.extra.weight"] = torch.zeros(3)
    t["model.layers.1.self_attn.q_proj.weight"] = torch.zeros(96, 96)
    t["model.norm.weight"] = torch.zeros(97)
    save_file(t, str(d / "model.safetensors"))
    with pytest.raises(WeightsError) as err:
        load_weights(_model(TINY_B), d, torch.float32, "cpu")
    e = err.value
    assert e.missing == ["lm_head.weight", "model.layers.2.self_attn.k_norm.weight"]
    assert e.unexpected == ["model.layers.0.mlp.extra.weight"]
    assert [(n, tuple(a), tuple(b)) for n, a, b in e.wrong_shape] == [
        ("model.layers.1.self_attn.q_proj.weight", (256, 96), (96, 96)),
        ("model.norm.weight", (96,), (97,))]
    msg = str(e)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)",
                   "expected (256, 96), found (96, 96)"):
        assert needle in msg


def test_folder_problems(tmp_path):
    with pytest.raises(FileNotFoundError):
        load_model(tmp_path / "absent", "float32", "cpu", ops=TorchOps())
    (tmp_path / "empty").mkdir()
    (tmp_path / "empty" / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(RuntimeError, match="No safetensors"):
        load_model(tmp_path / "empty", "float32", "cpu", ops=TorchOps())


def test_sharded_files_with_an_index(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_A, 0, torch.float32)
    t = load_file(str(d / "model.safetensors"))
    names = sorted(t)
    a, b = names[: len(names) // 2], names[len(names) // 2:]
    save_file({k: t[k] for k in a}, str(d / "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in b}, str(d / "model-00002-of-00002.safetensors"))
    (d / "model.safetensors").unlink()
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {
        **{k: "model-00001-of-00002.safetensors" for k in a},
        **{k: "model-00002-of-00002.safetensors" for k in b}}}))
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    assert torch.equal(model.final_norm.weight, t["model.norm.weight"])
