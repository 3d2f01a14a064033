"""Qwen3 dense as a `ModelSpec`.

Arrangement and tensor names: engine/models/qwen/_archs.py:92-125 (sizes there are
the 0.6B ones; here they come from config.json), engine/models/_builder.py:41-98 (one
position encoder shared by all layers, pre-norm blocks, tied or untied head) and the
checkpoint-name table of engine/models/qwen/_checkpoint.py:9-24.
"""

from __future__ import annotations

from tokensprint_amd.config.model_config import Qwen3Config
from tokensprint_amd.config.registry import register_architecture
from tokensprint_amd.models.spec import LayerSpec, ModelSpec, PartSpec, Run

ARCHITECTURE = "Qwen3ForCausalLM"


def qwen3_spec(cfg: Qwen3Config) -> ModelSpec:
    layers = []
    for i in range(cfg.num_layers):
        pre = f"model.layers.{i}."
        layers.append(LayerSpec(
            block="pre_norm",
            mixer=PartSpec("gqa_attention", {
                "prefix": pre + "self_attn.", "num_heads": cfg.num_heads,
                "num_kv_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
                "qk_norm": True, "qk_norm_eps": cfg.rms_norm_eps,
                "position": "rope", "window": cfg.layer_windows[i]}),
            feed_forward=PartSpec("swiglu", {
                "prefix": pre + "mlp.", "inner_dim": cfg.intermediate_size}),
            mixer_norm=PartSpec("rmsnorm", {
                "dim": cfg.hidden_size, "eps": cfg.rms_norm_eps,
                "weight": pre + "input_layernorm.weight"}),
            ffn_norm=PartSpec("rmsnorm", {
                "dim": cfg.hidden_size, "eps": cfg.rms_norm_eps,
                "weight": pre + "post_attention_layernorm.weight"}),
        ))
    embed_name = "model.embed_tokens.weight"
    if cfg.tie_word_embeddings:
        head = PartSpec("head", {"weight": embed_name, "vocab_size": cfg.vocab_size,
                                 "tied": True, "ignored": "lm_head.weight"})
    else:
        head = PartSpec("head", {"weight": "lm_head.weight", "vocab_size": cfg.vocab_size})
    return ModelSpec(
        architecture=ARCHITECTURE, width=cfg.hidden_size, vocab_size=cfg.vocab_size,
        embedding=PartSpec("embedding", {"weight": embed_name, "vocab_size": cfg.vocab_size}),
        positions={"rope": PartSpec("rope", {
            "dim": cfg.head_dim, "theta": cfg.rope_theta, "max_position": cfg.max_position})},
        layers=tuple(layers),
        order=tuple(Run(i) for i in range(cfg.num_layers)),
        final_norm=PartSpec("rmsnorm", {
            "dim": cfg.hidden_size, "eps": cfg.rms_norm_eps, "weight": "model.norm.weight"}),
        head=head, max_position=cfg.max_position, eos_token_id=cfg.eos_token_id,
    )


register_architecture(ARCHITECTURE, parse_config=Qwen3Config.from_dict, build_spec=qwen3_spec)
