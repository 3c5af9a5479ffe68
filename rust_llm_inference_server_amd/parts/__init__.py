"""The parts a model is put together from.  Importing the package registers the built-in
kinds: mixer ``attention``; feed-forward ``swiglu``; norm ``rmsnorm``; position ``rope`` and
``none``; block ``prenorm``; embedding ``token``; head ``linear``."""
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registration)
from .base import (Block, BuildContext, CacheBinding, CacheRequest, Embedding, FeedForward,
                   Head, Mixer, Norm, NormedInput, Part, PartSpec, PositionEncoding,
                   ResidualStream, TensorSpec, create, lookup, normed, project, register,
                   tensor_specs)

__all__ = ["Block", "BuildContext", "CacheBinding", "CacheRequest", "Embedding", "FeedForward",
           "Head", "Mixer", "Norm", "NormedInput", "Part", "PartSpec", "PositionEncoding",
           "ResidualStream", "TensorSpec", "create", "lookup", "normed", "project", "register",
           "tensor_specs"]
