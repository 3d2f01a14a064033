from tokensprint_amd.models import qwen3  # noqa: F401  (registers the architecture)
from tokensprint_amd.models.model import Model
from tokensprint_amd.models.spec import LayerSpec, ModelSpec, PartSpec, Run

__all__ = ["Model", "LayerSpec", "ModelSpec", "PartSpec", "Run"]
