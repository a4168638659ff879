"""Architectures: builders from a typed configuration to a ModelSpec, and the model that runs one."""
from . import llama  # registers the architecture
from .model import Model, load_model, random_model
from .spec import LayerCall, ModelSpec

__all__ = ["Model", "load_model", "random_model", "LayerCall", "ModelSpec"]
