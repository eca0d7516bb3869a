"""Checkpoint conversion: HF-style LLaMA / Baichuan state dicts to the key names
and tensor forms the operator classes take, and re-packing of int8 state dicts
that the reference saved.

Counterpart of convert_llama_weights (python/eet/transformers/modeling_llama.py:
739-784), convert_baichuan_weights (modeling_baichuan.py:572-602) and the
llama / baichuan tables of python/eet/utils/mapping.py:256-324.  Resulting keys:

    layer.N.self_attn.qkv_proj.{weight,scale}   fused [Q | K | V], [K=hidden, N=3*hidden]
    layer.N.self_attn.out_proj.{weight,scale}
    layer.N.self_attn.layernorm.weight
    layer.N.ffn.intermediate_0.{weight,scale}   gate_proj
    layer.N.ffn.intermediate_1.{weight,scale}   up_proj
    layer.N.ffn.output.{weight,scale}           down_proj
    layer.N.ffn.layernorm.weight
    embed_tokens.weight, norm.weight, lm_head.weight

'.weight' of a linear is int8 [K, N] in the gfx950 packed layout, '.scale' the
per-output-channel scales in the source dtype.
"""
import re

import torch

from . import ops
from ._lib import check, lib

LAYOUT_KEY = "__eet_layout__"
LAYOUT_GFX950_V1 = "gfx950-v1"
LAYOUT_REF_SM80 = "cutlass-sm80"

# HF sub-module name -> name under 'layer.N.' (mapping.py:256-296)
_RENAME = {
    "self_attn.q_proj": "self_attn.q_proj",
    "self_attn.k_proj": "self_attn.k_proj",
    "self_attn.v_proj": "self_attn.v_proj",
    "self_attn.qkv_proj": "self_attn.qkv_proj",
    "self_attn.W_pack": "self_attn.qkv_proj",          # Baichuan's fused projection
    "self_attn.o_proj": "self_attn.out_proj",
    "self_attn.rotary_emb.inv_freq": "self_attn.rotary_emb.inv_freq",
    "input_layernorm": "self_attn.layernorm",
    "mlp.gate_proj": "ffn.intermediate_0",
    "mlp.up_proj": "ffn.intermediate_1",
    "mlp.down_proj": "ffn.output",
    "post_attention_layernorm": "ffn.layernorm",
}

_LAYER_RE = re.compile(r"^(?:.*\.)?layers\.(\d+)\.(.+)\.(weight|bias|inv_freq)$")


def convert_name(key):
    """'model.layers.3.mlp.gate_proj.weight' -> 'layer.3.ffn.intermediate_0.weight';
    keys outside the layer stack lose their 'model.' prefix only."""
    m = _LAYER_RE.match(key)
    if m is None:
        return key[len("model."):] if key.startswith("model.") else key
    layer, sub, leaf = m.groups()
    if leaf == "inv_freq":
        sub, leaf = sub + ".inv_freq", None
    new = _RENAME.get(sub)
    if new is None:
        raise KeyError(f"unknown parameter '{key}'")
    return f"layer.{layer}.{new}" + (f".{leaf}" if leaf else "")


def _convert(model_dict, quant_mode, device=None):
    out = {LAYOUT_KEY: LAYOUT_GFX950_V1}
    # fuse q, k, v of every layer in that order (modeling_llama.py:745-753)
    qkv = {}
    work = {}
    for k, v in model_dict.items():
        nk = convert_name(k)
        m = re.match(r"^layer\.(\d+)\.self_attn\.([qkv])_proj\.weight$", nk)
        if m:
            qkv.setdefault(m.group(1), {})[m.group(2)] = v
        else:
            work[nk] = v
    for layer, parts in qkv.items():
        if set(parts) != {"q", "k", "v"}:
            raise KeyError(f"layer {layer}: q_proj / k_proj / v_proj must all be present")
        work[f"layer.{layer}.self_attn.qkv_proj.weight"] = torch.cat((parts["q"], parts["k"], parts["v"]), dim=0)
    for k, v in work.items():
        if k.startswith("layer.") and k.endswith(".weight") and v.dim() == 2:
            if device is not None:   # quantise and pack on the GPU; the results stay there
                w = v.detach().to(device).transpose(0, 1).contiguous()  # [in, out] = [K, N]
                if w.dtype not in (torch.float16, torch.float32):
                    w = w.float()
                processed, scale = ops.quant_weights_device(w, False, mode=quant_mode)
                del w
            else:
                w = v.detach().cpu().transpose(0, 1).contiguous()
                if w.dtype not in (torch.float16, torch.float32):
                    w = w.float()
                processed, scale = ops.quant_weights(w, torch.int8, False, mode=quant_mode)
            out[k] = processed
            out[k[: -len(".weight")] + ".scale"] = scale
        else:
            out[k] = v
    return out


def convert_llama_weights(model_dict, data_type=torch.int8, model_attr="model", quant_mode="ref128", device=None):
    """HF LLaMA state dict -> operator state dict (int8 weight-only).  With
    device="cuda:0" the linears are quantised and packed by the HIP packer and
    returned as GPU tensors (same bits as the host path)."""
    if data_type != torch.int8:
        raise NotImplementedError("[EET][ERROR] only the int8 weight-only conversion is implemented")
    return _convert(dict(model_dict), quant_mode, device)


def convert_baichuan_weights(model_dict, data_type=torch.int8, model_attr="model", quant_mode="ref128", device=None):
    """HF Baichuan state dict (fused W_pack) -> operator state dict (int8 weight-only); device as above."""
    if data_type != torch.int8:
        raise NotImplementedError("[EET][ERROR] only the int8 weight-only conversion is implemented")
    return _convert(dict(model_dict), quant_mode, device)


def repack_reference_state_dict(ref_dict):
    """An int8 state dict saved by the reference (torch.save of the converted
    dict, example/python/models/baichuan_transformers_example.py:42-46) holds
    every int8 '.weight' in the sm80 cutlass layout.  Undo that layout and pack
    for gfx950; everything else is passed through.  Scales are layout independent."""
    out = {LAYOUT_KEY: LAYOUT_GFX950_V1}
    L = lib()
    for k, v in ref_dict.items():
        if k == LAYOUT_KEY:
            continue
        if isinstance(v, torch.Tensor) and v.dtype == torch.int8 and v.dim() == 2:
            src = v.detach().cpu().contiguous()
            K, N = src.shape
            q = torch.empty_like(src)
            check(L.eet_unprocess_ref_sm80(src.data_ptr(), K, N, q.data_ptr()), "eet_unprocess_ref_sm80")
            out[k] = ops.pack_weights(q)
        else:
            out[k] = v
    return out


def check_layout(state_dict):
    tag = state_dict.get(LAYOUT_KEY, None)
    if tag is not None and tag != LAYOUT_GFX950_V1:
        raise RuntimeError(f"[EET][ERROR] state dict layout '{tag}' is not '{LAYOUT_GFX950_V1}'; "
                           "use repack_reference_state_dict for weights saved by the reference")
    if lib().eet_packed_layout_version() != 1:
        raise RuntimeError("[EET][ERROR] libeet_hip.so packs a different layout version")
