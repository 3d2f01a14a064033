"""Weights from safetensors by checkpoint tensor name.

Reading mirrors engine/models/_loader.py:54-76 (every *.safetensors file of the
folder, every key); there is no renaming step because parts declare the checkpoint's
own names.  All problems are reported in one error: missing names, unexpected names
and wrong shapes (the reference relies on load_state_dict(strict=True),
engine/models/_api.py:45).
"""

from __future__ import annotations

import json
import logging
from pathlib import Path

import torch
from safetensors import safe_open

from tokensprint_amd.parts.base import TensorDecl


log = logging.getLogger(__name__)


class WeightsError(RuntimeError):
    """The checkpoint does not hold exactly the tensors the model declares."""

    def __init__(self, missing, unexpected, wrong_shape):
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(
                f"{n}: expected {tuple(e)}, found {tuple(f)}" for n, e, f in wrong_shape))
        super().__init__("\n".join(lines))


class CheckpointFiles:
    """Names, shapes and lazy reads over the safetensors files of a model folder."""

    def __init__(self, model_dir) -> None:
        self.dir = Path(model_dir)
        if not self.dir.is_dir():
            raise FileNotFoundError(f"Failed to find model folder at {self.dir}.")
        index = self.dir / "model.safetensors.index.json"
        if index.is_file():
            names = sorted(set(json.loads(index.read_text())["weight_map"].values()))
            files = [self.dir / n for n in names]
        else:
            files = sorted(self.dir.glob("*.safetensors"))
        if not files:
            raise RuntimeError(f"No safetensors files found at {self.dir}.")
        self._where: dict[str, Path] = {}
        self._shape: dict[str, tuple[int, ...]] = {}
        for file in files:
            with safe_open(str(file), framework="pt", device="cpu") as f:
                for key in f.keys():
                    self._where[key] = file
                    self._shape[key] = tuple(f.get_slice(key).get_shape())

    def names(self):
        return list(self._where)

    def shape(self, name):
        return self._shape[name]

    def read(self, name) -> torch.Tensor:
        with safe_open(str(self._where[name]), framework="pt", device="cpu") as f:
            return f.get_tensor(name)


class TensorDict:
    """The same interface over tensors already in memory (random-weights mode)."""

    def __init__(self, tensors: dict[str, torch.Tensor]) -> None:
        self._t = tensors

    def names(self):
        return list(self._t)

    def shape(self, name):
        return tuple(self._t[name].shape)

    def read(self, name):
        return self._t[name]


def held_dtype(decl: TensorDecl, stored: torch.dtype, run_dtype: torch.dtype,
               cast_32bit: bool = False) -> torch.dtype:
    """The dtype a tensor is held in.

    Small vectors are held in float32 (exact for bfloat16 values) and integer
    tables in int32.  Matrices follow the run dtype, except that in a bfloat16 run
    a matrix the file stores in 32-bit stays 32-bit (its products then run on the
    float32 multiply-add kernels) unless `cast_32bit` asks for it to be rounded.
    """
    if decl.role == "table" or not stored.is_floating_point:
        return torch.int32
    if decl.role == "vector" or run_dtype == torch.float32:
        return torch.float32
    if (stored == torch.float32 or stored == torch.float64) and not cast_32bit:
        return torch.float32
    return torch.bfloat16


def check_tensors(decls: dict[str, TensorDecl], source) -> None:
    have = set(source.names())
    missing = sorted(n for n, d in decls.items() if n not in have and not d.optional)
    unexpected = sorted(have - set(decls))
    wrong = sorted((n, decls[n].shape, source.shape(n)) for n in have & set(decls)
                   if tuple(source.shape(n)) != tuple(decls[n].shape))
    if missing or unexpected or wrong:
        raise WeightsError(missing, unexpected, wrong)


def load_weights(model, source, run_dtype: torch.dtype, device, cast_32bit: bool = False) -> None:
    """Check `source` against the model's declarations, then hand the tensors over.

    `source` is a model folder path, a `CheckpointFiles` or a `TensorDict`.  In a bfloat16
    run matrices stored in 32-bit stay 32-bit, and a warning says how many and what that
    costs; `cast_32bit` rounds them to bfloat16 instead.
    """
    if isinstance(source, (str, Path)):
        source = CheckpointFiles(source)
    decls = model.tensor_decls()
    check_tensors(decls, source)
    have = set(source.names())
    needed = {n for part in model.parts() for n, d in part.tensors().items() if not d.optional}
    tensors, kept_wide = {}, []
    for name in sorted(needed & have):
        t = source.read(name)
        held = held_dtype(decls[name], t.dtype, run_dtype, cast_32bit)
        if held == torch.float32 and run_dtype != torch.float32 and decls[name].role == "matrix":
            kept_wide.append(name)
        tensors[name] = t.to(device=device, dtype=held).contiguous()
    if kept_wide:
        log.warning("%d matrices are stored in 32-bit and stay so in this bfloat16 run (%s, ...): "
                    "their products run on the float32 multiply-add kernels, many times slower "
                    "than the bfloat16 ones; load with cast_32bit=True (--cast-weights True) to "
                    "round them to bfloat16", len(kept_wide), kept_wide[0])
    model.load_tensors(tensors)
