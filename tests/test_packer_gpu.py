"""The packer on the GPU (eet_quantize_pack_device) against the known answers recorded from the reference,
the numpy oracle, and the shipped host packer: bit-exact in every case."""
import json
import os

import numpy as np
import pytest
import torch

import eet_amd
from oracle import quant as Q

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = json.load(open(os.path.join(HERE, "golden", "quant_known_answers.json")))


def golden_matrix(case, dtype=np.float32):
    K = case["K"]
    w = np.full((K, 64), 0.25, dtype)
    col = np.full(K, case["column"]["fill"], dtype)
    for k, v in case["column"]["set"].items():
        col[int(k)] = v
    w[:, 5] = col
    return w


@pytest.mark.parametrize("case", GOLD["quantize"], ids=lambda c: c["name"])
def test_known_answers(gpu, case):
    w = golden_matrix(case)
    q, p, s = eet_amd.quant_weights_device(torch.from_numpy(w).to(gpu), True)
    q, s = q.cpu().numpy(), s.cpu().numpy()
    assert float(s[5]) == case["scale"]
    if "q_all" in case:
        assert (q[:, 5] == case["q_all"]).all()
    for k, v in case.get("q", {}).items():
        assert int(q[int(k), 5]) == v, k
    assert torch.equal(p.cpu(), eet_amd.pack_weights(torch.from_numpy(q)))


def tricky(K, N, dtype, seed):
    """Random weights plus what a quantiser gets wrong first: an all-zero column, a column whose quotients
    sit exactly on .5 ties, one at the clamp (+absmax -> 128 -> 127, -absmax -> -128), tiny and huge columns."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    w[:, 1] = 0.0
    w[:, 2] = (rng.integers(-255, 256, K) * 0.5).astype(np.float32) / 128.0   # scale 1/128 once absmax is 1
    w[0, 2], w[1, 2] = 1.0, -1.0
    w[:, 3] = rng.choice([1.0, -1.0, 0.99609375, 0.00390625], K)
    w[:, 4] *= 1e-4
    w[:, 7] *= 3e3
    return w.astype(dtype)


@pytest.mark.parametrize("K,N", [(64, 16), (64, 144), (192, 400), (1024, 1040), (4096, 4096)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("mode", ["ref128", "sym127"])
def test_matches_host_packer(gpu, K, N, dtype, mode):
    w = torch.from_numpy(tricky(K, N, dtype, K + N))
    uh, ph, sh = eet_amd.quant_weights(w, torch.int8, True, mode=mode)
    ud, pd, sd = eet_amd.quant_weights_device(w.to(gpu), True, mode=mode)
    assert torch.equal(ud.cpu(), uh), "unprocessed int8"
    assert torch.equal(pd.cpu(), ph), "gfx950 layout"
    assert torch.equal(sd.cpu().view(torch.int16 if dtype == np.float16 else torch.int32),
                       sh.view(torch.int16 if dtype == np.float16 else torch.int32)), "scales (bit pattern)"
    p2, s2 = eet_amd.quant_weights_device(w.to(gpu), False, mode=mode)      # without the unprocessed output
    assert torch.equal(p2, pd) and torch.equal(s2, sd)
    if mode == "ref128" and K * N <= 1 << 20:
        qo, so = Q.quantize_ref128(w.numpy())
        assert np.array_equal(ud.cpu().numpy(), qo)


def test_full_size_properties(gpu):
    """LLaMA-7B gate projection (4096 x 11008) generated on the GPU: |q| <= 128, every non-zero column reaches
    127 or -128, dequantised error within half a step, and unpack(packed) == unprocessed."""
    g = torch.Generator(device=gpu).manual_seed(5)
    w = (torch.randn(4096, 11008, generator=g, device=gpu) * 0.02).half()
    q, p, s = eet_amd.quant_weights_device(w, True)
    assert torch.equal(eet_amd.unpack_weights(p.cpu()), q.cpu())
    ext = torch.maximum(q.amax(0), -q.amin(0) - 1)
    assert bool((ext == 127).all())
    s32 = w.float().abs().amax(0) / 128
    err = (q.float() * s32 - w.float()).abs()
    inside = (q > -128) & (q < 127)
    assert float((err[inside] / s32.expand_as(err)[inside]).max()) <= 0.5 + 1e-3


def test_arguments(gpu):
    from eet_amd._lib import lib
    L = lib()
    w = torch.zeros(64, 16, dtype=torch.float16, device=gpu)
    o = torch.zeros(64, 16, dtype=torch.int8, device=gpu)
    s = torch.zeros(16, dtype=torch.float16, device=gpu)
    ws = torch.zeros(16, dtype=torch.int32, device=gpu)
    ok = (w.data_ptr(), 1, 64, 16, 0, None, o.data_ptr(), s.data_ptr(), ws.data_ptr(), 64, None)
    assert L.eet_quantize_pack_device(*ok) == 0
    bad = list(ok); bad[2] = 96
    assert L.eet_quantize_pack_device(*bad) == -2          # K % 64
    bad = list(ok); bad[9] = 8
    assert L.eet_quantize_pack_device(*bad) == -4          # workspace too small
    bad = list(ok); bad[1] = 5
    assert L.eet_quantize_pack_device(*bad) == -1          # dtype
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):
        eet_amd.quant_weights_device(torch.zeros(64, 16))  # CPU tensor


def test_converter_on_device(gpu):
    """convert_llama_weights(device=...) quantises and packs with the HIP packer: same keys and bits as the
    host conversion, linears left on the GPU."""
    from eet_amd import convert
    hid, ff = 128, 192
    g = torch.Generator().manual_seed(3)
    r = lambda *s: (torch.randn(*s, generator=g) * 0.05).half()
    sd = {"model.embed_tokens.weight": r(50, hid), "model.norm.weight": r(hid), "lm_head.weight": r(50, hid)}
    p = "model.layers.0."
    for n in "qkvo":
        sd[p + f"self_attn.{n}_proj.weight"] = r(hid, hid)
    sd[p + "mlp.gate_proj.weight"], sd[p + "mlp.up_proj.weight"] = r(ff, hid), r(ff, hid)
    sd[p + "mlp.down_proj.weight"] = r(hid, ff)
    sd[p + "input_layernorm.weight"], sd[p + "post_attention_layernorm.weight"] = r(hid), r(hid)
    host = convert.convert_llama_weights(sd)
    dev = convert.convert_llama_weights(sd, device=gpu)
    assert host.keys() == dev.keys()
    for k, v in host.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(dev[k].cpu(), v), k
            if k.endswith("proj.weight") or k.startswith("layer.0.ffn.") and k.endswith(("weight", "scale")) and "layernorm" not in k:
                assert dev[k].device.type == "cuda", k
        else:
            assert dev[k] == v
