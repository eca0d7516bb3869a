"""The branches of the ops that LLaMA / Baichuan checkpoints never take, against the oracle, through the C ABI
and the operator classes: LayerNorm in place of RMSnorm, Q / K / V / output biases (BaichuanMmha), the output
bias and the post-layernorm tail of the gated feed-forward op, LayerNorm with a beta.
Reference: csrc/op/baichuan_mmha.cpp:45, 224-231, 295-297, 402; csrc/op/gated_ffn_int8.cpp:139-146, 328-357."""
import numpy as np
import pytest
import torch

from eet_amd import decoder as D
from eet_amd import ops
from eet_amd._lib import check, lib
from oracle import ops as O

from gpu_util import assert_close, stream

pytestmark = pytest.mark.gpu

EPS = 1e-5


@pytest.mark.parametrize("M,N", [(1, 64), (7, 4096), (33, 5120), (3, 16384)])
def test_layernorm_and_bias_kernels(gpu, M, N):
    L = lib()
    g = torch.Generator().manual_seed(M + N)
    x = (torch.randn(M, N, generator=g) * 1.5 + 0.7).half()
    inp = torch.randn(M, N, generator=g).half()
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).half()
    beta = (0.2 * torch.randn(N, generator=g)).half()
    bias = torch.randn(N, generator=g).half()
    xd, gd, bd, id_, biasd = [t.to(gpu) for t in (x, gamma, beta, inp, bias)]
    out = torch.empty_like(xd)
    check(L.eet_layernorm(xd.data_ptr(), gd.data_ptr(), bd.data_ptr(), out.data_ptr(), M, N, EPS, stream()))
    assert_close(out.cpu().numpy(), O.layernorm(x.numpy(), gamma.numpy(), beta.numpy(), EPS), 1e-2, 1e-3, "layernorm")
    o2 = xd.clone()
    check(L.eet_add_bias(o2.data_ptr(), biasd.data_ptr(), M, N, stream()))
    assert np.array_equal(o2.cpu().numpy(), O.add_bias(x.numpy(), bias.numpy()))          # one fp16 add: bit-exact
    o3 = xd.clone()
    check(L.eet_add_bias_residual_norm(o3.data_ptr(), id_.data_ptr(), biasd.data_ptr(), gd.data_ptr(), bd.data_ptr(),
                                       M, N, EPS, stream()))
    assert_close(o3.cpu().numpy(), O.add_bias_residual_norm(x.numpy(), inp.numpy(), bias.numpy(), gamma.numpy(),
                                                           beta.numpy(), EPS), 1e-2, 1e-3, "post-LN tail with bias")
    o4 = xd.clone()
    check(L.eet_add_bias_residual_norm(o4.data_ptr(), id_.data_ptr(), None, gd.data_ptr(), None, M, N, EPS, stream()))
    assert_close(o4.cpu().numpy(), O.add_bias_residual_norm(x.numpy(), inp.numpy(), None, gamma.numpy(), None, EPS),
                 1e-2, 1e-3, "post-LN tail without bias (RMSnorm)")
    assert L.eet_layernorm(xd.data_ptr(), gd.data_ptr(), None, out.data_ptr(), M, N, EPS, stream()) == -1
    assert L.eet_add_bias(o2.data_ptr(), biasd.data_ptr(), M, 12, stream()) == -2


def desc(hidden, heads, d_ff, batch=3, prompt=12, cap=24):
    return ops.MetaDesc(dtype=torch.float16, batch_size=batch, head_num=heads, hidden_units=hidden, layer_num=1,
                        max_seq_len=prompt, max_full_seq_len=cap, activation_fn="silu", d_kv=0, d_ff=d_ff,
                        cuda_device="cuda:0", layernorm_eps=EPS, is_int8=True)


def linear(K, N, g):
    w = (torch.randn(K, N, generator=g) * 0.05).half()
    u, p, s = ops.quant_weights(w, torch.int8, True)
    return u.numpy(), s.numpy(), p, s


def test_baichuan_attention_with_biases(gpu):
    hidden, heads = 256, 4
    dh = hidden // heads
    g = torch.Generator().manual_seed(8)
    qkv_u, qkv_s, qkv_p, qkv_st = linear(hidden, 3 * hidden, g)
    o_u, o_s, o_p, o_st = linear(hidden, hidden, g)
    gamma = (1 + 0.1 * torch.randn(hidden, generator=g)).half()
    beta = (0.2 * torch.randn(hidden, generator=g)).half()
    qb, kb, vb = [(0.3 * torch.randn(hidden, generator=g)).half() for _ in range(3)]
    ob = (0.3 * torch.randn(hidden, generator=g)).half()
    d = desc(hidden, heads, 704)
    ops.workspaces.clear()
    op = ops.BaichuanMmha(d, qkv_p.to(gpu), qkv_st.to(gpu), qb.to(gpu), kb.to(gpu), vb.to(gpu), o_p.to(gpu),
                          o_st.to(gpu), ob.to(gpu), gamma.to(gpu), beta.to(gpu))
    ref = O.OracleAttention(3, heads, dh, 24, qkv_u, qkv_s, o_u, o_s, gamma.numpy(), EPS, rope=False,
                            qkv_bias=torch.cat((qb, kb, vb)).numpy(), o_bias=ob.numpy(), beta=beta.numpy())
    B, S = 3, 7
    e = torch.empty(0, dtype=torch.long)
    x = (torch.randn(B, S, hidden, generator=g) + 0.3).half()
    y = op.forward(x.to(gpu), e, e, True, True, True, D.alibi_mask(heads, S).to(gpu))
    want = ref.forward(x.numpy(), None, True, O.alibi_mask(heads, S))
    assert_close(y.cpu().numpy(), want, 2e-2, 4e-3, "biased attention prefill")
    for t in range(3):
        step = S + t + 1
        x1 = (torch.randn(B, 1, hidden, generator=g) + 0.3).half()
        y = op.forward(x1.to(gpu), e, e, True, True, False, D.alibi_mask(heads, step)[:, -1:, :].contiguous().to(gpu))
        want = ref.forward(x1.numpy(), None, False, O.alibi_bias(heads, step))
        assert_close(y.cpu().numpy(), want, 2e-2, 4e-3, f"biased attention step {step}")
    assert_close(op.k_cache[:, :, :step].cpu().numpy(), ref.k_cache[:, :, :step], 4e-3, 4e-3, "k cache (with bias)")
    # only the output bias: the unbiased front, bias behind the residual
    op2 = ops.BaichuanMmha(d, qkv_p.to(gpu), qkv_st.to(gpu), e, e, e, o_p.to(gpu), o_st.to(gpu), ob.to(gpu),
                           gamma.to(gpu), e)
    ref2 = O.OracleAttention(3, heads, dh, 24, qkv_u, qkv_s, o_u, o_s, gamma.numpy(), EPS, rope=False, o_bias=ob.numpy())
    y = op2.forward(x.to(gpu), e, e, True, True, True, D.alibi_mask(heads, S).to(gpu))
    assert_close(y.cpu().numpy(), ref2.forward(x.numpy(), None, True, O.alibi_mask(heads, S)), 2e-2, 4e-3, "output bias only")
    x1 = torch.randn(B, 1, hidden, generator=g).half()
    y = op2.forward(x1.to(gpu), e, e, True, True, False, D.alibi_mask(heads, S + 1)[:, -1:, :].contiguous().to(gpu))
    assert_close(y.cpu().numpy(), ref2.forward(x1.numpy(), None, False, O.alibi_bias(heads, S + 1)), 2e-2, 4e-3,
                 "output bias only, step")
    # the rotary op refuses Q / K / V biases for fp16, as the reference's split kernel does; partial sets are refused
    with pytest.raises(NotImplementedError, match="biases are not supported with fp16"):
        ops.LlamaMmha(d, qkv_p.to(gpu), qkv_st.to(gpu), qb.to(gpu), kb.to(gpu), vb.to(gpu), o_p.to(gpu), o_st.to(gpu),
                      ob.to(gpu), gamma.to(gpu), beta.to(gpu))
    with pytest.raises(RuntimeError, match="all must be given"):
        ops.BaichuanMmha(d, qkv_p.to(gpu), qkv_st.to(gpu), qb.to(gpu), e, vb.to(gpu), o_p.to(gpu), o_st.to(gpu), e,
                         gamma.to(gpu), beta.to(gpu))
    ops.workspaces.clear()


@pytest.mark.parametrize("M_rows", [(2, 1), (3, 9), (3, 12)])
def test_ffn_bias_layernorm_and_post_layernorm(gpu, M_rows):
    B, S = M_rows
    hidden, d_ff = 256, 704
    g = torch.Generator().manual_seed(B * 31 + S)
    gu, gs, gp, gst = linear(hidden, d_ff, g)
    uu, us, up, ust = linear(hidden, d_ff, g)
    du, ds, dp, dst = linear(d_ff, hidden, g)
    gamma = (1 + 0.1 * torch.randn(hidden, generator=g)).half()
    beta = (0.2 * torch.randn(hidden, generator=g)).half()
    ob = (0.3 * torch.randn(hidden, generator=g)).half()
    junk = torch.randn(d_ff, generator=g).half()        # intermediate biases: accepted, never used
    d = desc(hidden, 4, d_ff)
    e = torch.empty(0)
    x = (torch.randn(B, S, hidden, generator=g) + 0.4).half()
    ops.workspaces.clear()
    for lb, obias in [(beta, ob), (None, ob), (beta, None), (None, None)]:
        op = ops.GatedFeedForwardNetworkInt8(d, gp.to(gpu), gst.to(gpu), junk.to(gpu), up.to(gpu), ust.to(gpu),
                                             junk.to(gpu), dp.to(gpu), dst.to(gpu),
                                             obias.to(gpu) if obias is not None else e, gamma.to(gpu),
                                             lb.to(gpu) if lb is not None else e)
        ref = O.OracleFFN(gu, gs, uu, us, du, ds, gamma.numpy(), EPS, beta=lb.numpy() if lb is not None else None,
                          o_bias=obias.numpy() if obias is not None else None)
        for pre_ln, add_res in [(True, True), (True, False), (False, True), (False, False)]:
            what = f"beta={lb is not None} o_bias={obias is not None} pre_layernorm={pre_ln} add_residual={add_res}"
            if add_res and not pre_ln and obias is not None and lb is None:
                with pytest.raises(RuntimeError, match="needs layernorm_bias"):
                    op.forward(x.to(gpu), pre_ln, add_res)
                continue
            y = op.forward(x.to(gpu), pre_ln, add_res)
            assert_close(y.cpu().numpy(), ref.forward(x.numpy(), pre_ln, add_res), 2e-2, 4e-3, what)
    # LayerNorm op with a beta
    ln = ops.LayerNorm(d, gamma.to(gpu), beta.to(gpu))
    assert_close(ln.layer_norm(x.to(gpu)).cpu().numpy(),
                 O.layernorm(x.numpy().reshape(B * S, hidden), gamma.numpy(), beta.numpy(), EPS).reshape(B, S, hidden),
                 1e-2, 1e-3, "LayerNorm op")
    ops.workspaces.clear()
