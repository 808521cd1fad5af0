"""Model assembly.  Importing this package registers the built-in architecture."""

from mini_infer_amd.models import llama  # noqa: F401
from mini_infer_amd.models.decoder import DecoderModel
from mini_infer_amd.models.spec import Architecture, LayerCall, LayerSpec, ModelSpec
from mini_infer_amd.registry import ARCHITECTURES


def architecture_for(raw_config: dict) -> Architecture:
    """The registered architecture a raw config.json names in `architectures[0]`."""
    names = raw_config.get("architectures") or []
    if not names:
        raise ValueError("config.json has no `architectures`; cannot choose a model")
    return ARCHITECTURES.lookup(str(names[0]))


__all__ = [
    "Architecture",
    "DecoderModel",
    "LayerCall",
    "LayerSpec",
    "ModelSpec",
    "architecture_for",
]
