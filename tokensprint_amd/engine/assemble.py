"""From a model folder to a loaded model: config.json chooses the architecture.

Counterpart of engine/models/_api.py:31-59 (config -> build -> load weights), minus
tokenizer and download.  `ops` is the kernel provider; None means the HIP kernels,
which raise if no GPU or no compiler-built library is there.
"""

from __future__ import annotations

import torch

from tokensprint_amd.config.model_config import architecture_of, read_config_json
from tokensprint_amd.config.registry import get_architecture
from tokensprint_amd.models.model import Model
from tokensprint_amd.parts.base import BuildContext
from tokensprint_amd.weights.loader import TensorDict, load_weights

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
          "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype must be bfloat16 or float32, got {name}")
        return name
    if name not in DTYPES:
        raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {name!r}")
    return DTYPES[name]


def build_model(raw_config: dict, dtype, device, ops=None):
    """(typed config, Model without weights) for a raw config.json dict."""
    dtype = parse_dtype(dtype)
    device = torch.device(device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", 0)
    if ops is None:
        from tokensprint_amd.kernels import load_hip_ops
        ops = load_hip_ops(device)
    arch = get_architecture(architecture_of(raw_config))
    config = arch.parse_config(raw_config)
    spec = arch.build_spec(config)
    ctx = BuildContext(ops=ops, dtype=dtype, device=device, width=spec.width)
    return config, Model(spec, ctx)


def load_model(model_dir, dtype="bfloat16", device="cuda:0", ops=None, cast_32bit=False):
    """(typed config, Model with weights) from a folder with config.json and safetensors.
    `cast_32bit`: in a bfloat16 run, round matrices the files store in 32-bit to bfloat16
    (by default they stay 32-bit and are served by the float32 kernels)."""
    config, model = build_model(read_config_json(model_dir), dtype, device, ops)
    load_weights(model, model_dir, model.ctx.dtype, model.ctx.device, cast_32bit=cast_32bit)
    return config, model


def random_model(raw_config: dict, seed: int, dtype="bfloat16", device="cuda:0", ops=None,
                 std: float = 0.02):
    """A model with random weights made directly in memory (no folder is written)."""
    from tokensprint_amd.weights.random_init import random_tensors
    config, model = build_model(raw_config, dtype, device, ops)
    tensors = random_tensors(raw_config, seed, dtype=model.ctx.dtype, std=std,
                             device=model.ctx.device)
    load_weights(model, TensorDict(tensors), model.ctx.dtype, model.ctx.device)
    return config, model
