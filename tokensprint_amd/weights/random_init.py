"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has no such mode (its norm weights start as torch.empty,
engine/nn/base_layers.py:35).  Matrices are N(0, std) and norm vectors
1 + U(-0.1, 0.1); every tensor has its own generator keyed by (seed, name), so the
values do not depend on the order tensors are made in.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch
from safetensors.torch import save_file

from tokensprint_amd.config.model_config import architecture_of
from tokensprint_amd.config.registry import get_architecture
from tokensprint_amd.parts.base import BuildContext

_DTYPE_NAMES = {torch.bfloat16: "bfloat16", torch.float32: "float32"}


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def declared_tensors(raw_config: dict):
    """name -> TensorDecl for the architecture config.json names (no device needed)."""
    from tokensprint_amd.models.model import Model

    arch = get_architecture(architecture_of(raw_config))
    spec = arch.build_spec(arch.parse_config(raw_config))
    ctx = BuildContext(ops=None, dtype=torch.float32, device=torch.device("cpu"),
                       width=spec.width)
    return Model(spec, ctx).tensor_decls()


def random_tensors(raw_config: dict, seed: int, dtype=torch.float32, std: float = 0.02,
                   device="cpu") -> dict[str, torch.Tensor]:
    out = {}
    for name, decl in sorted(declared_tensors(raw_config).items()):
        if decl.optional:
            continue
        gen = torch.Generator(device=device).manual_seed(_tensor_seed(seed, name))
        if decl.role == "vector":
            t = 1.0 + (torch.rand(decl.shape, generator=gen, device=device) * 0.2 - 0.1)
        elif decl.role == "table":
            raise ValueError(f"no random rule for integer table {name}")
        else:
            t = torch.randn(decl.shape, generator=gen, device=device) * std
        out[name] = t.to(dtype)
    return out


def write_random_model(model_dir, raw_config: dict, seed: int, dtype=torch.float32,
                       std: float = 0.02, device="cpu") -> Path:
    """Write config.json and model.safetensors; returns the folder.  `device` is where the
    values are drawn (a GPU draws a large model's in a second; its generator gives other
    values than the CPU's for the same seed)."""
    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    cfg = dict(raw_config)
    cfg["torch_dtype"] = _DTYPE_NAMES[dtype]
    tensors = random_tensors(cfg, seed, dtype=dtype, std=std, device=device)
    (model_dir / "config.json").write_text(json.dumps(cfg, indent=2))
    save_file({k: v.cpu().contiguous() for k, v in tensors.items()},
              str(model_dir / "model.safetensors"))
    return model_dir
