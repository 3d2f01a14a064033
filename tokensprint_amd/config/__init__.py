from tokensprint_amd.config.engine_config import Config, SamplingParams
from tokensprint_amd.config.model_config import ConfigError, Qwen3Config, read_config_json
from tokensprint_amd.config.registry import (
    all_registered_models,
    all_registered_repo_ids,
    architecture_names,
    get_architecture,
    get_model_family,
    get_model_repo_id,
    get_models_from_family,
    load_named_config,
    lookup,
    models_by_family,
    model_is_registered,
    register_architecture,
    register_named_model,
    resolve_model_name,
)

__all__ = [
    "Config", "SamplingParams", "ConfigError", "Qwen3Config", "read_config_json",
    "all_registered_models", "all_registered_repo_ids", "architecture_names",
    "get_architecture", "get_model_family", "get_model_repo_id",
    "get_models_from_family", "load_named_config", "lookup", "models_by_family", "model_is_registered",
    "register_architecture", "register_named_model", "resolve_model_name",
]
