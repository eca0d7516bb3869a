"""The operator classes (LlamaMmha, BaichuanMmha, GatedFeedForwardNetworkInt8, LayerNorm) and the
decoder built from them, against the oracle's composition of the same ops.

The composed outputs pass through several fp16 buffers; the tolerance against the oracle is
2e-2 relative / 4e-3 absolute on O(1) activations (per-op parity is held to 1e-2 / 1e-3 elsewhere)."""
import numpy as np
import pytest
import torch

import eet_amd
from eet_amd import decoder as D
from oracle import ops as O

from gpu_util import assert_close

pytestmark = pytest.mark.gpu

RT, AT = 2e-2, 4e-3


def tiny_cfg(alibi=False, layers=2, hidden=256):
    return D.DecoderConfig(num_layers=layers, hidden=hidden, heads=4, d_ff=704, vocab=512, eps=1e-6, alibi=alibi,
                           max_batch=3, max_prompt=12, max_full_seq=24)


def oracle_decoder(cfg, sd, raw):
    layers = []
    dh = cfg.hidden // cfg.heads
    for i in range(cfg.num_layers):
        pre = f"layer.{i}."
        n = lambda k: (raw[pre + k][0].numpy(), raw[pre + k][1].numpy())
        attn = O.OracleAttention(cfg.max_batch, cfg.heads, dh, cfg.max_full_seq, *n("self_attn.qkv_proj"),
                                 *n("self_attn.out_proj"), sd[pre + "self_attn.layernorm.weight"].numpy(), cfg.eps,
                                 rope=not cfg.alibi)
        ffn = O.OracleFFN(*n("ffn.intermediate_0"), *n("ffn.intermediate_1"), *n("ffn.output"),
                          sd[pre + "ffn.layernorm.weight"].numpy(), cfg.eps)
        layers.append((attn, ffn))
    return O.OracleDecoder(sd["embed_tokens.weight"].numpy(), layers, sd["norm.weight"].numpy(),
                           sd["lm_head.weight"].numpy(), cfg.eps, n_head=cfg.heads, alibi=cfg.alibi)


@pytest.mark.parametrize("alibi,hidden", [(False, 256), (True, 256), (False, 384), (True, 384)])   # head size 64, 96
def test_single_layer_ops(gpu, alibi, hidden):
    cfg = tiny_cfg(alibi, layers=1, hidden=hidden)
    sd, raw = D.random_state_dict(cfg, seed=5)
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    ref = oracle_decoder(cfg, sd, raw)
    attn, ffn = model.layers[0]
    oattn, offn = ref.layers[0]
    g = torch.Generator().manual_seed(1)
    B, S = 3, 7
    x = torch.randn(B, S, cfg.hidden, generator=g).half()
    pad = torch.tensor([[0], [2], [0]])
    e = torch.empty(0, dtype=torch.long)
    bias_full = D.alibi_mask(cfg.heads, S) if alibi else None
    y = attn.forward(x.to(gpu), pad.to(gpu) if not alibi else e, e, True, True, True,
                     bias_full.to(gpu) if alibi else torch.empty(0))
    want = oattn.forward(x.numpy(), None if alibi else pad.numpy().reshape(-1), True,
                         O.alibi_mask(cfg.heads, S) if alibi else None)
    assert_close(y.cpu().numpy(), want, RT, AT, "attention prefill")
    z = ffn.forward(y, True, True)
    wantz = offn.forward(want)
    assert_close(z.cpu().numpy(), wantz, RT, AT, "ffn prefill")
    # incremental steps
    for t in range(3):
        x1 = torch.randn(B, 1, cfg.hidden, generator=g).half()
        step = S + t + 1
        bias = D.alibi_mask(cfg.heads, step)[:, -1:, :].contiguous() if alibi else None
        y = attn.forward(x1.to(gpu), pad.to(gpu) if not alibi else e, e, True, True, False,
                         bias.to(gpu) if alibi else torch.empty(0))
        want = oattn.forward(x1.numpy(), None if alibi else pad.numpy().reshape(-1), False,
                             O.alibi_bias(cfg.heads, step) if alibi else None)
        assert_close(y.cpu().numpy(), want, RT, AT, f"attention step {t}")
        assert attn.step == oattn.step == step
    # the cache now holds the oracle's rows
    assert_close(attn.k_cache[:, :, :step].cpu().numpy(), oattn.k_cache[:, :, :step], 4e-3, 4e-3, "k cache")
    # output buffers are shared by name across ops of the same kind, as in the reference
    y2 = attn.forward(x1.to(gpu), e, e, True, True, True, bias_full[:, :1, :1].to(gpu) if alibi else torch.empty(0))
    assert y2.data_ptr() == y.data_ptr()


def test_final_layernorm_op(gpu):
    cfg = tiny_cfg()
    desc = eet_amd.MetaDesc(torch.float16, 2, cfg.heads, cfg.hidden, 1, 8, 16, "silu", 0, cfg.d_ff, "cuda:0",
                            False, 1e-5, True)
    g = torch.Generator().manual_seed(2)
    gamma = (1 + 0.1 * torch.randn(cfg.hidden, generator=g)).half()
    ln = eet_amd.LayerNorm(desc, gamma.to(gpu), torch.empty(0))
    x = torch.randn(2, 5, cfg.hidden, generator=g).half()
    assert_close(ln.layer_norm(x.to(gpu)).cpu().numpy(), O.rmsnorm(x.numpy(), gamma.numpy(), 1e-5), 2e-3, 1e-3)


def test_op_validation(gpu):
    cfg = tiny_cfg(layers=1)
    sd, _ = D.random_state_dict(cfg, seed=6)
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    attn, ffn = model.layers[0]
    e = torch.empty(0, dtype=torch.long)
    with pytest.raises(RuntimeError, match="batch"):
        attn.forward(torch.zeros(4, 1, cfg.hidden, dtype=torch.float16, device=gpu), e, e, True, True, True)
    with pytest.raises(RuntimeError, match="prompt length"):
        attn.forward(torch.zeros(1, 13, cfg.hidden, dtype=torch.float16, device=gpu), e, e, True, True, True)
    attn.forward(torch.zeros(1, 12, cfg.hidden, dtype=torch.float16, device=gpu), e, e, True, True, True)
    for _ in range(12):
        attn.forward(torch.zeros(1, 1, cfg.hidden, dtype=torch.float16, device=gpu), e, e, True, True, False)
    with pytest.raises(RuntimeError, match="max_full_seq_len"):
        attn.forward(torch.zeros(1, 1, cfg.hidden, dtype=torch.float16, device=gpu), e, e, True, True, False)
    with pytest.raises(RuntimeError, match="seq_len 1"):
        attn.forward(torch.zeros(1, 2, cfg.hidden, dtype=torch.float16, device=gpu), e, e, True, True, False)
    with pytest.raises(RuntimeError, match="reorder_state"):
        attn.forward(torch.zeros(1, 1, cfg.hidden, dtype=torch.float16, device=gpu), e,
                     torch.zeros(1, dtype=torch.long), True, True, False)          # CPU tensor
    with pytest.raises(RuntimeError, match="fp16"):
        ffn.forward(torch.zeros(1, 1, cfg.hidden, device=gpu), True, True)


@pytest.mark.parametrize("alibi", [False, True])
def test_greedy_tokens_match_oracle(gpu, alibi):
    """Prefill + 6 greedy steps on a tiny random model: token-for-token equality with the CPU
    oracle decoder wherever the oracle's own top-2 logit margin exceeds the numeric noise."""
    cfg = tiny_cfg(alibi)
    sd, raw = D.random_state_dict(cfg, seed=7)
    # larger head weights so that the logits are well separated
    sd["lm_head.weight"] = sd["lm_head.weight"] * 8
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    ref = oracle_decoder(cfg, sd, raw)
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, cfg.vocab, (3, 9), generator=g)
    logits = ref.step(ids.numpy(), True)
    got = model.logits(ids.to(gpu), True).float().cpu().numpy()[:, 0]
    n_checked = 0
    for t in range(6):
        assert_close(got, logits, 3e-2, 3e-2, f"logits step {t}")
        top2 = np.sort(logits, -1)[:, -2:]
        nxt = logits.argmax(-1)
        for b in range(3):
            if top2[b, 1] - top2[b, 0] > 0.1:
                assert got[b].argmax() == nxt[b]
                n_checked += 1
        logits = ref.step(nxt[:, None], False)
        got = model.logits(torch.from_numpy(nxt)[:, None].to(gpu), False).float().cpu().numpy()[:, 0]
    assert n_checked >= 9
    # and the loop helper itself
    model2 = D.Int8Decoder(cfg, sd, device="cuda:0")
    toks = model2.greedy(ids.to(gpu), 4).cpu().numpy()
    assert toks.shape == (3, 4)


def test_converted_checkpoint_runs(gpu):
    """HF-named fp16 LLaMA weights -> convert_llama_weights -> Int8Decoder, against an oracle
    decoder whose int8 weights come from the oracle's own quantiser on the same fp16 matrices."""
    from eet_amd import convert
    from oracle import quant as oq
    cfg = tiny_cfg(False)
    g = torch.Generator().manual_seed(11)
    r = lambda *s: (torch.randn(*s, generator=g) * 0.02).half()
    H, F = cfg.hidden, cfg.d_ff
    hf = {"model.embed_tokens.weight": r(cfg.vocab, H), "model.norm.weight": 1 + 5 * r(H),
          "lm_head.weight": 8 * r(cfg.vocab, H)}
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}."
        for n in "qkvo":
            hf[p + f"self_attn.{n}_proj.weight"] = r(H, H)
        hf[p + "mlp.gate_proj.weight"], hf[p + "mlp.up_proj.weight"] = r(F, H), r(F, H)
        hf[p + "mlp.down_proj.weight"] = r(H, F)
        hf[p + "input_layernorm.weight"], hf[p + "post_attention_layernorm.weight"] = 1 + 5 * r(H), 1 + 5 * r(H)
    sd = convert.convert_llama_weights(hf, torch.int8)
    model = D.Int8Decoder(cfg, sd, device="cuda:0")

    def oq_lin(w_hf):
        q, s = oq.quantize_ref128(w_hf.t().contiguous().numpy())
        return torch.from_numpy(q), torch.from_numpy(s)
    raw = {}
    for i in range(cfg.num_layers):
        p, pre = f"model.layers.{i}.", f"layer.{i}."
        raw[pre + "self_attn.qkv_proj"] = oq_lin(torch.cat([hf[p + f"self_attn.{n}_proj.weight"] for n in "qkv"], 0))
        raw[pre + "self_attn.out_proj"] = oq_lin(hf[p + "self_attn.o_proj.weight"])
        raw[pre + "ffn.intermediate_0"] = oq_lin(hf[p + "mlp.gate_proj.weight"])
        raw[pre + "ffn.intermediate_1"] = oq_lin(hf[p + "mlp.up_proj.weight"])
        raw[pre + "ffn.output"] = oq_lin(hf[p + "mlp.down_proj.weight"])
    ref = oracle_decoder(cfg, sd, raw)
    ids = torch.randint(0, cfg.vocab, (2, 7), generator=g)
    logits = ref.step(ids.numpy(), True)
    got = model.logits(ids.to(gpu), True).float().cpu().numpy()[:, 0]
    assert_close(got, logits, 3e-2, 3e-2, "prefill logits")
    nxt = logits.argmax(-1)
    logits = ref.step(nxt[:, None], False)
    got = model.logits(torch.from_numpy(nxt)[:, None].to(gpu), False).float().cpu().numpy()[:, 0]
    assert_close(got, logits, 3e-2, 3e-2, "decode logits")

    # a dict carrying the reference's layout tag is refused rather than mis-read
    bad = dict(sd)
    bad[convert.LAYOUT_KEY] = convert.LAYOUT_REF_SM80
    with pytest.raises(RuntimeError, match="layout"):
        D.Int8Decoder(cfg, bad, device="cuda:0")


@pytest.mark.parametrize("alibi", [False, True])
def test_beam_search_reorder(gpu, alibi):
    """reorder_state on incremental calls: beam b continues from the cache rows of beam
    reorder_state[b] (llama_mmha.cpp:248-252), including a beam that is dropped and one taken twice."""
    cfg = tiny_cfg(alibi, layers=1)
    sd, raw = D.random_state_dict(cfg, seed=9)
    attn = D.Int8Decoder(cfg, sd, device="cuda:0").layers[0][0]
    oattn = oracle_decoder(cfg, sd, raw).layers[0][0]
    g = torch.Generator().manual_seed(4)
    B, S = 3, 5
    e = torch.empty(0, dtype=torch.long)
    x = torch.randn(B, S, cfg.hidden, generator=g).half()
    attn.forward(x.to(gpu), e, e, True, True, True, D.alibi_mask(cfg.heads, S).to(gpu) if alibi else torch.empty(0))
    oattn.forward(x.numpy(), None, True, O.alibi_mask(cfg.heads, S) if alibi else None)
    orders = [None, [2, 0, 0], [1, 1, 2], None, [0, 2, 1]]
    for t, order in enumerate(orders):
        step = S + t + 1
        x1 = torch.randn(B, 1, cfg.hidden, generator=g).half()
        bias = D.alibi_mask(cfg.heads, step)[:, -1:, :].contiguous().to(gpu) if alibi else torch.empty(0)
        ro = torch.tensor(order, dtype=torch.long, device=gpu) if order is not None else e
        y = attn.forward(x1.to(gpu), e, ro, True, True, False, bias)
        want = oattn.forward(x1.numpy(), None, False, O.alibi_bias(cfg.heads, step) if alibi else None, reorder=order)
        assert_close(y.cpu().numpy(), want, RT, AT, f"attention step {t} order {order}")
    assert_close(attn.k_cache[:, :, :step].cpu().numpy(), oattn.k_cache[:, :, :step], 4e-3, 4e-3, "k cache")
    assert_close(attn.v_cache[:, :, :step].cpu().numpy(), oattn.v_cache[:, :, :step], 4e-3, 4e-3, "v cache")
    with pytest.raises(RuntimeError, match="reorder_state"):
        attn.forward(x1.to(gpu), e, torch.tensor([0, 1, 2], dtype=torch.int32, device=gpu), True, True, False,
                     D.alibi_mask(cfg.heads, step + 1)[:, -1:, :].contiguous().to(gpu) if alibi else torch.empty(0))


@pytest.mark.parametrize("alibi,eos", [(False, None), (True, None), (False, 7)])
def test_beam_search_driver(gpu, alibi, eos):
    """Int8Decoder.beam_search (the caller of reorder_state: generation.py:1564-1580) against the oracle
    decoder's beam search: the same sequences, scores within the logits' tolerance; one beam is greedy."""
    cfg = D.DecoderConfig(num_layers=2, hidden=256, heads=4, d_ff=704, vocab=64, eps=1e-6, alibi=alibi, max_batch=6,
                          max_prompt=12, max_full_seq=24)
    sd, raw = D.random_state_dict(cfg, seed=27)
    sd["lm_head.weight"] = sd["lm_head.weight"] * 8          # separates the candidates' scores
    ids = torch.randint(0, cfg.vocab, (2, 6), generator=torch.Generator().manual_seed(12))
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    ref = oracle_decoder(cfg, sd, raw)
    toks, scores = model.beam_search(ids.to(gpu), 3, 9, eos_token_id=eos, pad_token_id=0)
    want_t, want_s = ref.beam_search(ids.numpy(), 3, 9, eos=eos, pad_token=0)
    assert np.array_equal(toks.numpy(), want_t), (toks, want_t)
    assert np.abs(scores.numpy() - want_s).max() < 2e-2
    assert model.reorder_state.numel() == 0                   # the driver leaves no reorder behind
    one, _ = model.beam_search(ids.to(gpu), 1, 5)
    assert torch.equal(one, D.Int8Decoder(cfg, sd, device="cuda:0").greedy(ids.to(gpu), 5).cpu())
    with pytest.raises(RuntimeError, match="exceeds max_batch"):
        model.beam_search(ids.to(gpu), 4, 3)


@pytest.mark.parametrize("alibi", [False, True])
def test_left_padded_batch(gpu, alibi):
    """attention_mask with left padding -> pre_padding_len (modeling_llama.py:276-279): prefill and
    three decode steps against the oracle decoder; the last position of every sequence is a real token."""
    cfg = tiny_cfg(alibi)
    sd, raw = D.random_state_dict(cfg, seed=21)
    sd["lm_head.weight"] = sd["lm_head.weight"] * 8
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    ref = oracle_decoder(cfg, sd, raw)
    g = torch.Generator().manual_seed(8)
    B, S = 3, 10
    ids = torch.randint(0, cfg.vocab, (B, S), generator=g)
    pads = [0, 4, 7]
    mask = torch.ones(B, S, dtype=torch.long)
    for b, p in enumerate(pads):
        mask[b, :p] = 0
    pad_np = np.array(pads, dtype=np.int64)
    logits = ref.step(ids.numpy(), True, pad_np)
    got = model.logits(ids.to(gpu), True, mask.to(gpu)).float().cpu().numpy()[:, 0]
    for t in range(3):
        assert_close(got, logits, 3e-2, 3e-2, f"logits step {t}")
        nxt = logits.argmax(-1)
        logits = ref.step(nxt[:, None], False, pad_np)
        got = model.logits(torch.from_numpy(nxt)[:, None].to(gpu), False, mask.to(gpu)).float().cpu().numpy()[:, 0]
    assert_close(got, logits, 3e-2, 3e-2, "logits last step")


@pytest.mark.parametrize("alibi", [False, True])
def test_decode_with_more_than_32_sequences(gpu, alibi):
    """40 sequences per step: past the row count of the fused decode calls, so the ops issue RMSnorm, the
    MFMA-tile GEMMs (with the split-k workspace), attention and the residual epilogue one by one."""
    cfg = D.DecoderConfig(num_layers=1, hidden=256, heads=4, d_ff=704, vocab=512, eps=1e-6, alibi=alibi,
                          max_batch=40, max_prompt=6, max_full_seq=12)
    sd, raw = D.random_state_dict(cfg, seed=11)
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    ref = oracle_decoder(cfg, sd, raw)
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(0, cfg.vocab, (40, 5), generator=g)
    logits = ref.step(ids.numpy(), True)
    got = model.logits(ids.to(gpu), True).float().cpu().numpy()[:, 0]
    for t in range(3):
        assert_close(got, logits, 3e-2, 3e-2, f"logits step {t}")
        nxt = logits.argmax(-1)
        logits = ref.step(nxt[:, None], False)
        got = model.logits(torch.from_numpy(nxt)[:, None].to(gpu), False).float().cpu().numpy()[:, 0]


def hf_model_from_state(cfg, sd, raw):
    """The independent float64 model (tests/hf_formulation.py) over the dequantised weights of an
    EET-named state dict; fused QKV columns are [Q | K | V] (modeling_llama.py:85)."""
    import hf_formulation as HF
    assert not cfg.alibi or cfg.heads & (cfg.heads - 1) == 0
    slopes = HF.power_of_two_slopes(cfg.heads) if cfg.alibi else None
    H = cfg.hidden

    def deq(name):
        q, s = raw[name]
        return (q.numpy().astype(np.float64) * s.numpy().astype(np.float64)[None, :]).T      # [out, in]
    layers = []
    for i in range(cfg.num_layers):
        pre = f"layer.{i}."
        qkv = deq(pre + "self_attn.qkv_proj")
        layers.append(HF.Layer(qkv[:H], qkv[H:2 * H], qkv[2 * H:], deq(pre + "self_attn.out_proj"),
                               deq(pre + "ffn.intermediate_0"), deq(pre + "ffn.intermediate_1"), deq(pre + "ffn.output"),
                               sd[pre + "self_attn.layernorm.weight"].numpy(), sd[pre + "ffn.layernorm.weight"].numpy(),
                               cfg.heads, cfg.eps, slopes))
    return HF.Model(sd["embed_tokens.weight"].numpy(), layers, sd["norm.weight"].numpy(),
                    sd["lm_head.weight"].numpy(), cfg.eps)


@pytest.mark.parametrize("alibi", [False, True])
def test_decoder_matches_hf_formulation(gpu, alibi):
    """The product against the independently written float64 model without a KV cache (teacher
    forced: prefill 6 tokens, then 4 incremental calls), so a mistake shared by ops.py and the
    oracle's composition would still show.  Error is relative to the RMS of the logits; the
    product rounds to fp16 between ops, the independent model never does."""
    cfg = tiny_cfg(alibi)
    sd, raw = D.random_state_dict(cfg, seed=31)
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    hf = hf_model_from_state(cfg, sd, raw)
    ids = torch.randint(0, cfg.vocab, (3, 10), generator=torch.Generator().manual_seed(5))
    want = hf.logits(ids.numpy())
    rms = np.sqrt((want * want).mean())
    got = model.logits(ids[:, :6].to(gpu), True).float().cpu().numpy()[:, 0]
    assert np.abs(got - want[:, 5]).max() / rms < 2e-2
    for t in range(6, 10):
        got = model.logits(ids[:, t:t + 1].to(gpu), False).float().cpu().numpy()[:, 0]
        assert np.abs(got - want[:, t]).max() / rms < 2e-2, t


@pytest.mark.parametrize("name", ["llama7b", "baichuan13b"])
def test_full_width_layer(gpu, name):
    """One decoder layer at the real width of benchmark configurations 4 and 5 (4096 / 32 heads /
    11008 at batch 8; 5120 / 40 heads / 13696 with ALiBi at batch 32): a short prompt and two
    incremental calls through the operator classes, against the oracle layer.
    With K up to 13696 behind fp16 intermediates that the product and the oracle round at
    different points, a handful of the ~10^5 outputs sit 2 fp16 steps apart at magnitude 4-8;
    the per-element bound here is 2e-2 relative / 1e-2 absolute, backed by an RMS error bound
    of 3e-3 over the tensor -- one to two fp16 steps of outputs of magnitude 1-4, which is what
    two correct roundings of nearly equal fp32 values differ by (every linear of these shapes is held to 1e-2 / 1e-3 on its own in
    test_gemm_gpu.py and test_config_shapes_gpu.py)."""
    def close(got, want, what):
        assert_close(got, want, 2e-2, 1e-2, what)
        err = np.asarray(got, np.float32) - np.asarray(want, np.float32)
        assert float(np.sqrt((err * err).mean())) < 3e-3, what
    if name == "llama7b":
        cfg = D.DecoderConfig(num_layers=1, hidden=4096, heads=32, d_ff=11008, vocab=64, alibi=False, max_batch=8,
                              max_prompt=8, max_full_seq=12)
    else:
        cfg = D.DecoderConfig(num_layers=1, hidden=5120, heads=40, d_ff=13696, vocab=64, alibi=True, max_batch=32,
                              max_prompt=8, max_full_seq=12)
    eet_amd.ops.workspaces.clear()
    sd, raw = D.random_state_dict(cfg, seed=41)
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    ref = oracle_decoder(cfg, sd, raw)
    attn, ffn = model.layers[0]
    oattn, offn = ref.layers[0]
    g = torch.Generator().manual_seed(2)
    B, S = cfg.max_batch, 5
    e = torch.empty(0, dtype=torch.long)
    x = torch.randn(B, S, cfg.hidden, generator=g).half()
    print(f"full-width layer {name}: prefill B={B} S={S}", flush=True)
    bias = D.alibi_mask(cfg.heads, S).to(gpu) if cfg.alibi else torch.empty(0)
    y = attn.forward(x.to(gpu), e, e, True, True, True, bias)
    want = oattn.forward(x.numpy(), None, True, O.alibi_mask(cfg.heads, S) if cfg.alibi else None)
    close(y.cpu().numpy(), want, "attention prefill")
    z = ffn.forward(y, True, True)
    close(z.cpu().numpy(), offn.forward(y.cpu().numpy()), "ffn prefill")     # same input to both
    for t in range(2):
        step = S + t + 1
        x1 = torch.randn(B, 1, cfg.hidden, generator=g).half()
        print(f"full-width layer {name}: incremental call, step {step}", flush=True)
        bias = D.alibi_mask(cfg.heads, step)[:, -1:, :].contiguous().to(gpu) if cfg.alibi else torch.empty(0)
        y = attn.forward(x1.to(gpu), e, e, True, True, False, bias)
        want = oattn.forward(x1.numpy(), None, False, O.alibi_bias(cfg.heads, step) if cfg.alibi else None)
        close(y.cpu().numpy(), want, f"attention step {step}")
        z = ffn.forward(y, True, True)
        close(z.cpu().numpy(), offn.forward(y.cpu().numpy()), f"ffn step {step}")
    del model
    eet_amd.ops.workspaces.clear()
    torch.cuda.empty_cache()
