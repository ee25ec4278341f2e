"""Models: a configuration becomes a `DecoderModel` (every architecture here is a decoder made
of registered parts; what differs between architectures is their configuration class)."""
from ..config.base import ModelConfig
from .decoder import CachePlan, DecoderModel


def build_model_description(config: ModelConfig) -> DecoderModel:
    """The model as parts and declarations, before any weight or device memory."""
    from .. import parts  # noqa: F401  (registers the built-in parts)
    return DecoderModel(config)


__all__ = ["CachePlan", "DecoderModel", "build_model_description"]
