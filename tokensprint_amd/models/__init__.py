from tokensprint_amd.models import palelix, pinedra, qwen3, zolorax, zonopel  # noqa: F401  (register the architectures)
from tokensprint_amd.models.model import Model
from tokensprint_amd.models.spec import LayerSpec, ModelSpec, PartSpec, Run

__all__ = ["Model", "LayerSpec", "ModelSpec", "PartSpec", "Run"]
