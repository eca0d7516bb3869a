"""eet_amd: MI355X (gfx950) implementation of EET's int8 weight-only linear
path -- offline packer, fused dequant-GEMM, masked decode attention -- behind
the reference's own operator API."""
from .ops import (BaichuanMmha, CrossMultiHeadAttention, Embedding, FeedForwardNetwork,  # noqa: F401
                  GatedFeedForwardNetwork, GatedFeedForwardNetworkInt8, LayerNorm, LlamaMmha,
                  MaskedMultiHeadAttention, MetaDesc, MultiHeadAttention, pack_weights,
                  pack_weights_torch, preprocess_weights, quant_weights, quant_weights_torch,
                  unpack_weights)

__version__ = "0.1.0"
