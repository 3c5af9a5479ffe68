"""Models as data (``ModelSpec``) and the architectures that ship with the package."""
from .llama import llama_spec
from .spec import LayerSpec, Model, ModelSpec, RunEntry

__all__ = ["LayerSpec", "Model", "ModelSpec", "RunEntry", "llama_spec"]
