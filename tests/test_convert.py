"""Checkpoint converter: key names and tensors of convert_llama_weights /
convert_baichuan_weights (python/eet/transformers/modeling_llama.py:739-784,
modeling_baichuan.py:572-602, python/eet/utils/mapping.py:256-324), and the
re-packing of int8 weights saved in the reference's sm80 layout.  CPU only."""
import numpy as np
import pytest
import torch

from eet_amd import convert, ops
from oracle import quant as oq

HID, FF, VOCAB, LAYERS = 128, 192, 50, 2


def _hf_llama(seed=0, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: (torch.randn(*s, generator=g) * 0.05).to(dtype)
    sd = {"model.embed_tokens.weight": r(VOCAB, HID), "model.norm.weight": r(HID), "lm_head.weight": r(VOCAB, HID)}
    for i in range(LAYERS):
        p = f"model.layers.{i}."
        for n in "qkvo":
            sd[p + f"self_attn.{n}_proj.weight"] = r(HID, HID)
        sd[p + "self_attn.rotary_emb.inv_freq"] = torch.arange(4).float()
        sd[p + "mlp.gate_proj.weight"] = r(FF, HID)
        sd[p + "mlp.up_proj.weight"] = r(FF, HID)
        sd[p + "mlp.down_proj.weight"] = r(HID, FF)
        sd[p + "input_layernorm.weight"] = r(HID)
        sd[p + "post_attention_layernorm.weight"] = r(HID)
    return sd


def _hf_baichuan(seed=0):
    sd = _hf_llama(seed)
    for i in range(LAYERS):
        p = f"model.layers.{i}.self_attn."
        sd[p + "W_pack.weight"] = torch.cat([sd.pop(p + f"{n}_proj.weight") for n in "qkv"], 0)
        sd.pop(p + "rotary_emb.inv_freq")
    return sd


# The names the reference's model classes read from the converted dict
# (modeling_llama.py:64-75, 119-131, 601-627).
EXPECTED_LAYER_KEYS = {
    "self_attn.qkv_proj.weight", "self_attn.qkv_proj.scale", "self_attn.out_proj.weight", "self_attn.out_proj.scale",
    "self_attn.layernorm.weight", "ffn.intermediate_0.weight", "ffn.intermediate_0.scale",
    "ffn.intermediate_1.weight", "ffn.intermediate_1.scale", "ffn.output.weight", "ffn.output.scale",
    "ffn.layernorm.weight",
}


@pytest.mark.parametrize("key,want", [
    ("model.layers.0.self_attn.q_proj.weight", "layer.0.self_attn.q_proj.weight"),
    ("model.layers.11.self_attn.o_proj.weight", "layer.11.self_attn.out_proj.weight"),
    ("model.layers.3.self_attn.W_pack.weight", "layer.3.self_attn.qkv_proj.weight"),
    ("layers.3.self_attn.qkv_proj.weight", "layer.3.self_attn.qkv_proj.weight"),
    ("model.layers.7.input_layernorm.weight", "layer.7.self_attn.layernorm.weight"),
    ("model.layers.7.post_attention_layernorm.weight", "layer.7.ffn.layernorm.weight"),
    ("model.layers.2.mlp.gate_proj.weight", "layer.2.ffn.intermediate_0.weight"),
    ("model.layers.2.mlp.up_proj.weight", "layer.2.ffn.intermediate_1.weight"),
    ("model.layers.2.mlp.down_proj.weight", "layer.2.ffn.output.weight"),
    ("model.layers.2.self_attn.rotary_emb.inv_freq", "layer.2.self_attn.rotary_emb.inv_freq"),
    ("model.embed_tokens.weight", "embed_tokens.weight"),
    ("model.norm.weight", "norm.weight"),
    ("lm_head.weight", "lm_head.weight"),
])
def test_convert_name(key, want):
    assert convert.convert_name(key) == want


def test_convert_name_unknown():
    with pytest.raises(KeyError):
        convert.convert_name("model.layers.0.self_attn.mystery.weight")


def _check_linear(out, name, w_hf):
    """w_hf is the HF [out, in] matrix; converted weight must be the packed
    quantisation of its transpose, bit for bit."""
    w = w_hf.transpose(0, 1).contiguous()
    q_want, s_want = oq.quantize_ref128(w.numpy())
    assert out[name + ".weight"].dtype == torch.int8 and tuple(out[name + ".weight"].shape) == tuple(w.shape)
    got_q = ops.unpack_weights(out[name + ".weight"]).numpy()
    np.testing.assert_array_equal(got_q, q_want)
    assert out[name + ".scale"].dtype == w.dtype
    np.testing.assert_array_equal(out[name + ".scale"].numpy().view(np.uint16 if w.dtype == torch.float16 else np.uint32),
                                  s_want.view(np.uint16 if w.dtype == torch.float16 else np.uint32))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_convert_llama(dtype):
    hf = _hf_llama(1, dtype)
    out = convert.convert_llama_weights(hf, torch.int8)
    assert out.pop(convert.LAYOUT_KEY) == convert.LAYOUT_GFX950_V1
    for i in range(LAYERS):
        got = {k[len(f"layer.{i}."):] for k in out if k.startswith(f"layer.{i}.")}
        assert got == EXPECTED_LAYER_KEYS | {"self_attn.rotary_emb.inv_freq"}
        p = f"model.layers.{i}."
        fused = torch.cat([hf[p + f"self_attn.{n}_proj.weight"] for n in "qkv"], 0)
        _check_linear(out, f"layer.{i}.self_attn.qkv_proj", fused)
        _check_linear(out, f"layer.{i}.self_attn.out_proj", hf[p + "self_attn.o_proj.weight"])
        _check_linear(out, f"layer.{i}.ffn.intermediate_0", hf[p + "mlp.gate_proj.weight"])
        _check_linear(out, f"layer.{i}.ffn.intermediate_1", hf[p + "mlp.up_proj.weight"])
        _check_linear(out, f"layer.{i}.ffn.output", hf[p + "mlp.down_proj.weight"])
        assert torch.equal(out[f"layer.{i}.self_attn.layernorm.weight"], hf[p + "input_layernorm.weight"])
        assert torch.equal(out[f"layer.{i}.ffn.layernorm.weight"], hf[p + "post_attention_layernorm.weight"])
    # outside the layer stack: untouched fp tensors, 'model.' stripped
    assert torch.equal(out["embed_tokens.weight"], hf["model.embed_tokens.weight"])
    assert torch.equal(out["norm.weight"], hf["model.norm.weight"])
    assert torch.equal(out["lm_head.weight"], hf["lm_head.weight"])
    assert not any(k.startswith("model.") for k in out)


def test_convert_baichuan_equals_llama_on_same_weights():
    a = convert.convert_llama_weights(_hf_llama(2), torch.int8)
    b = convert.convert_baichuan_weights(_hf_baichuan(2), torch.int8)
    a = {k: v for k, v in a.items() if "rotary_emb" not in k}
    assert set(a) == set(b)
    for k in a:
        if isinstance(a[k], torch.Tensor):
            assert torch.equal(a[k], b[k]), k


def test_convert_missing_projection():
    hf = _hf_llama(3)
    del hf["model.layers.1.self_attn.k_proj.weight"]
    with pytest.raises(KeyError):
        convert.convert_llama_weights(hf, torch.int8)


def test_convert_rejects_other_types():
    with pytest.raises(NotImplementedError):
        convert.convert_llama_weights(_hf_llama(4), torch.float16)


def test_repack_reference_state_dict():
    """A dict as the reference saves it: int8 weights in the sm80 layout (built
    here with the oracle's restatement of that layout), scales, fp16 norms."""
    rng = np.random.default_rng(5)
    ref, want = {}, {}
    for name, (K, N) in {"layer.0.self_attn.qkv_proj": (128, 384), "layer.0.ffn.output": (192, 128)}.items():
        q = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ref[name + ".weight"] = torch.from_numpy(np.ascontiguousarray(oq.preprocess_ref_sm80(q)).view(np.int8).reshape(K, N))
        ref[name + ".scale"] = torch.from_numpy(rng.random(N).astype(np.float16))
        want[name + ".weight"] = ops.pack_weights(torch.from_numpy(q))
    ref["norm.weight"] = torch.ones(128, dtype=torch.float16)
    out = convert.repack_reference_state_dict(ref)
    assert out[convert.LAYOUT_KEY] == convert.LAYOUT_GFX950_V1
    for k, v in want.items():
        assert torch.equal(out[k], v), k
    for k in ref:
        if not k.endswith(".weight") or ref[k].dtype != torch.int8:
            assert out[k] is ref[k]


def test_check_layout():
    convert.check_layout({convert.LAYOUT_KEY: convert.LAYOUT_GFX950_V1})
    convert.check_layout({})
    with pytest.raises(RuntimeError):
        convert.check_layout({convert.LAYOUT_KEY: convert.LAYOUT_REF_SM80})
