"""Drop-in for the reference's pybind11 extension module `EET`
(csrc/py11/eet2py.cpp): `from EET import MetaDesc, LlamaMmha, ...` in the
reference's unchanged python/eet model code resolves to the gfx950 ops."""
from eet_amd.ops import (BaichuanMmha, CrossMultiHeadAttention, Embedding, FeedForwardNetwork,  # noqa: F401
                         GatedFeedForwardNetwork, GatedFeedForwardNetworkInt8, LayerNorm, LlamaMmha,
                         MaskedMultiHeadAttention, MetaDesc, MultiHeadAttention, preprocess_weights,
                         quant_weights)

__version__ = "dev"
