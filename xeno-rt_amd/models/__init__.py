"""A model as data: its parts, and the order in which its layers run."""
from .decoder import DecoderModel, LayerCall, ModelSpec

__all__ = ["DecoderModel", "LayerCall", "ModelSpec"]
