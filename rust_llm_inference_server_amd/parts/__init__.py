"""The parts a model is put together from.  Importing the package registers the built-in
kinds: mixers ``attention``, ``latent_attention``, ``time_mix``, ``gated_delta``,
``selective_scan`` and ``parallel``; feed-forwards ``swiglu``, ``clamped_glu`` and
``routed_swiglu``; norms ``rmsnorm`` and ``layernorm``; position ``rope`` and ``none``; blocks
``prenorm`` and ``parallel``; embedding ``token``; head ``linear``."""
from . import attention, block, embedding, latent, mlp, norm, recurrent, rope  # noqa: F401  (registration)
from .base import (Block, BuildContext, CacheBinding, CacheRequest, Embedding, FeedForward,
                   Head, Mixer, Norm, NormedInput, Part, PartSpec, PositionEncoding,
                   ResidualStream, TensorSpec, create, lookup, normed, project, register,
                   tensor_specs)

__all__ = ["Block", "BuildContext", "CacheBinding", "CacheRequest", "Embedding", "FeedForward",
           "Head", "Mixer", "Norm", "NormedInput", "Part", "PartSpec", "PositionEncoding",
           "ResidualStream", "TensorSpec", "create", "lookup", "normed", "project", "register",
           "tensor_specs"]
