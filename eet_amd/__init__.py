"""eet_amd: MI355X (gfx950) implementation of EET's int8 weight-only linear
path -- offline packer, fused dequant-GEMM, masked decode attention -- behind
the reference's own operator API."""
from .ops import (BaichuanMmha, CrossMultiHeadAttention, Embedding, FeedForwardNetwork,  # noqa: F401
                  GatedFeedForwardNetwork, GatedFeedForwardNetworkInt8, LayerNorm, LlamaMmha,
                  MaskedMultiHeadAttention, MetaDesc, MultiHeadAttention, pack_weights,
                  pack_weights_torch, preprocess_weights, quant_weights, quant_weights_device, quant_weights_torch,
                  unpack_weights)

from .convert import (convert_baichuan_weights, convert_llama_weights, convert_name,  # noqa: F401
                      repack_reference_state_dict)

__version__ = "0.1.0"
