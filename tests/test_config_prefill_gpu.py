"""Prefill at the real sizes of benchmark configurations 4 and 5, through the C ABI.

(i)   Configuration 4's prefill GEMMs at M = 8 * 1024 = 8192 rows (QKV 4096 -> 12288, O 4096 -> 4096,
      gate|up 4096 -> 2 * 11008 with the SwiGLU epilogue, down 11008 -> 4096 with the residual epilogue):
      every output element against an fp32 dequantise-then-matmul computed on the GPU with torch, and a
      seeded 512-row subset against the CPU oracle.
(ii)  eet_prefill_attention on the grids those prompts launch (B = 8, H = 32, S = 1024; B = 8, H = 40,
      S = 2048 with the ALiBi table): with one key repeated along the sequence the score of every key is the
      same, so context row i is the softmax(bias[:i+1])-weighted mean of V[:i+1] -- computed in fp32 on the
      GPU for every (b, h, i); and with random keys, four (b, h) pairs against the CPU oracle.
(iii) One LLaMA-7B-width layer (4096 / 32 heads / 11008) with a 1024-token prompt at batch 2 through the
      operator classes, against the oracle layer (the prompt path: RMSnorm kernel, large-M GEMMs,
      qkv split + rotary + cache write, flash prefill attention).
Tolerance: 1e-2 relative / 1e-3 absolute for the GEMMs and the attention kernel (the SwiGLU epilogue
3e-3 absolute against the composition that never rounds gate and up); the composed layer as in
test_layer_gpu.test_full_width_layer."""
import numpy as np
import pytest
import torch

import eet_amd
from eet_amd import decoder as D
from eet_amd import ops
from eet_amd._lib import check, lib
from oracle import ops as O

from gpu_util import assert_close, gemm_fused, stream

pytestmark = pytest.mark.gpu

HIDDEN, DFF, M_PROMPT = 4096, 11008, 8192


def device_linear(K, N, seed, gpu):
    """(unprocessed int8 [K, N], packed, scales) on the GPU, from the device packer (bit-identical to the host's)."""
    g = torch.Generator(device=gpu).manual_seed(seed)
    w = (torch.randn(K, N, generator=g, device=gpu) * 0.02).half()
    q, p, s = ops.quant_weights_device(w, True)
    return q, p, s


def assert_close_gpu(got, want, rtol, atol, what):
    err = (got.float() - want).abs()
    bad = err > atol + rtol * want.abs()
    n_bad = int(bad.sum())
    assert n_bad == 0, f"{what}: {n_bad} of {bad.numel()} outside tolerance, max err {float(err.max()):.5f}"
    return float(err.max())


@pytest.mark.parametrize("name,K,N,epi", [("qkv", HIDDEN, 3 * HIDDEN, 0), ("o", HIDDEN, HIDDEN, 1),
                                          ("gate|up+swiglu", HIDDEN, 2 * DFF, 2), ("down", DFF, HIDDEN, 1)])
def test_config4_prefill_gemm_every_row(gpu, name, K, N, epi):
    M = M_PROMPT
    g = torch.Generator(device=gpu).manual_seed(K + N)
    x = torch.randn(M, K, generator=g, device=gpu).half()
    res = torch.randn(M, N, generator=g, device=gpu).half() if epi == 1 else None
    print(f"config 4 prefill {name}: M={M} K={K} N={N}", flush=True)
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(7))[:512].sort().values
    if epi == 2:
        F = N // 2
        qg, pg, sg = device_linear(K, F, 1, gpu)
        qu, pu, su = device_linear(K, F, 2, gpu)
        w01, s01 = ops.interleave_gate_up(pg, sg, pu, su)
        got = gemm_fused(x, w01, s01, M, N, K, 2)
        x32 = x.float()
        gate = (x32 @ (qg.float() * sg.float()[None, :]))
        up = (x32 @ (qu.float() * su.float()[None, :]))
        want = up * gate / (1 + torch.exp(-gate))
        worst = assert_close_gpu(got, want, 1e-2, 3e-3, name)
        xs = x[rows.to(gpu)].cpu().numpy()
        ref = O.swiglu(O.dequant_matmul(xs, qg.cpu().numpy(), sg.cpu().numpy()),
                       O.dequant_matmul(xs, qu.cpu().numpy(), su.cpu().numpy()))
        assert_close(got[rows.to(gpu)].cpu().numpy(), ref, rtol=1e-2, atol=1e-3, what=name + " (oracle rows)")
    else:
        q, p, s = device_linear(K, N, 3 + epi, gpu)
        got = gemm_fused(x, p, s, M, N, K, epi, res)
        want = x.float() @ (q.float() * s.float()[None, :])
        if epi == 1:
            want = want.half().float() + res.float()       # fp16 add of the rounded product
        worst = assert_close_gpu(got, want, 1e-2, 2e-3 if epi == 1 else 1e-3, name)
        xs = x[rows.to(gpu)].cpu().numpy()
        ref = O.dequant_matmul(xs, q.cpu().numpy(), s.cpu().numpy())
        if epi == 1:
            ref = O.residual_add(ref, res[rows.to(gpu)].cpu().numpy())
        assert_close(got[rows.to(gpu)].cpu().numpy(), ref, rtol=1e-2, atol=2e-3 if epi == 1 else 1e-3,
                     what=name + " (oracle rows)")
    print(f"  max abs err over all {M} x {N if epi != 2 else N // 2} outputs: {worst:.2e}", flush=True)
    # size-independent property on all rows: doubling the scales doubles the plain product exactly
    if epi == 0:
        got2 = gemm_fused(x, p, (s.float() * 2).half(), M, N, K, 0)
        assert ((got2.float() - 2 * got.float()).abs() <= 2.0 ** -23).all()


def prefill_attention(q, kc, vc, S, alibi=None, pad=None):
    B, H, T, dh = kc.shape
    ctx = torch.empty(B, S, H * dh, dtype=torch.float16, device=kc.device)
    check(lib().eet_prefill_attention(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), ctx.data_ptr(),
                                      alibi.data_ptr() if alibi is not None else None,
                                      pad.data_ptr() if pad is not None else None, B, H, S, dh, T, stream()),
          "eet_prefill_attention")
    return ctx


def alibi_table(H, S, gpu):
    """[H, S] fp16: slope_h * j, as the decoder hands it to the op (the last row of the reference's mask)."""
    slopes = torch.tensor(D.alibi_slopes(H), dtype=torch.float32)
    return (slopes[:, None] * torch.arange(S, dtype=torch.float32)[None, :]).half().to(gpu)


@pytest.mark.parametrize("B,H,S,alibi", [(8, 32, 1024, False), (8, 40, 2048, True), (8, 40, 2048, False),
                                         (1, 32, 8192, False), (1, 8, 6001, True)])   # the last two: past the reference's 4096 / 2048 caps
def test_prefill_attention_full_grid_uniform_keys(gpu, B, H, S, alibi):
    """Every (b, h, i) of the launch the configuration makes.  All keys of a (b, h) pair are the same row, so
    the scores of a query are equal and its weights are softmax(bias[:i+1]) (uniform without a bias)."""
    dh = 128
    g = torch.Generator(device=gpu).manual_seed(S + H)
    q = torch.randn(B, H, S, dh, generator=g, device=gpu).half()
    krow = torch.randn(B, H, 1, dh, generator=g, device=gpu).half()
    kc = krow.expand(B, H, S, dh).contiguous()
    vc = torch.randn(B, H, S, dh, generator=g, device=gpu).half()
    table = alibi_table(H, S, gpu) if alibi else None
    print(f"prefill attention, uniform keys: B={B} H={H} S={S} alibi={alibi}", flush=True)
    got = prefill_attention(q, kc, vc, S, table).view(B, S, H, dh)
    worst = 0.0
    for h in range(H):
        b16 = table[h].float() if alibi else torch.zeros(S, device=gpu)
        # the bias grows with j, so the row maximum over j <= i is b[i]: w[i, j] = exp(b[j] - b[i]) for j <= i
        w = torch.exp(b16[None, :] - b16[:, None]).tril()
        w = w / (w.sum(-1, keepdim=True) + 1e-6)
        want = torch.einsum("ij,bjd->bid", w, vc[:, h].float())
        worst = max(worst, assert_close_gpu(got[:, :, h], want, 1e-2, 1e-3, f"head {h}"))
    print(f"  max abs err over all {B * H * S} rows: {worst:.2e}", flush=True)


@pytest.mark.parametrize("B,H,S,alibi", [(8, 32, 1024, False), (8, 40, 2048, True)])
def test_prefill_attention_full_grid_against_oracle(gpu, B, H, S, alibi):
    """Random q, k, v on the full grid; four (b, h) pairs, among them the first and the last workgroup
    column, against the CPU oracle."""
    dh = 128
    g = torch.Generator(device=gpu).manual_seed(S * 3 + H)
    q, kc, vc = [torch.randn(B, H, S, dh, generator=g, device=gpu).half() for _ in range(3)]
    table = alibi_table(H, S, gpu) if alibi else None
    print(f"prefill attention vs oracle: B={B} H={H} S={S} alibi={alibi}", flush=True)
    got = prefill_attention(q, kc, vc, S, table).view(B, S, H, dh)
    torch.cuda.synchronize()
    for b, h in [(0, 0), (B - 1, H - 1), (3, 17), (5, H // 2)]:
        bias = None
        if alibi:
            row = table[h].float().cpu().numpy()
            bias = np.where(np.arange(S)[None, :] > np.arange(S)[:, None], -np.inf, row[None, :])[None].astype(np.float32)
        want = O.prefill_attention(q[b:b + 1, h:h + 1].cpu().numpy(), kc[b:b + 1, h:h + 1].cpu().numpy(),
                                   vc[b:b + 1, h:h + 1].cpu().numpy(), None, bias)
        assert_close(got[b, :, h].cpu().numpy(), want[0], what=f"(b, h) = ({b}, {h})")


def test_full_width_layer_long_prompt(gpu):
    """LLaMA-7B width, batch 2, 1024-token prompt: M = 2048 rows through the prompt path of both ops, then
    one incremental call, against the oracle layer."""
    from test_layer_gpu import oracle_decoder

    def close(got, want, what):
        assert_close(got, want, 2e-2, 1e-2, what)
        err = np.asarray(got, np.float32) - np.asarray(want, np.float32)
        rms = float(np.sqrt((err * err).mean()))
        print(f"  {what}: max abs err {np.abs(err).max():.2e}, rms err {rms:.2e}", flush=True)
        assert rms < 3e-3, what
    cfg = D.DecoderConfig(num_layers=1, hidden=HIDDEN, heads=32, d_ff=DFF, vocab=64, alibi=False, max_batch=2,
                          max_prompt=1024, max_full_seq=1030)
    ops.workspaces.clear()
    sd, raw = D.random_state_dict(cfg, seed=43)
    model = D.Int8Decoder(cfg, sd, device="cuda:0")
    ref = oracle_decoder(cfg, sd, raw)
    attn, ffn = model.layers[0]
    oattn, offn = ref.layers[0]
    g = torch.Generator().manual_seed(4)
    B, S = 2, 1024
    e = torch.empty(0, dtype=torch.long)
    x = torch.randn(B, S, cfg.hidden, generator=g).half()
    print(f"full-width layer, long prompt: B={B} S={S}", flush=True)
    y = attn.forward(x.to(gpu), e, e, True, True, True, torch.empty(0))
    want = oattn.forward(x.numpy(), None, True, None)
    close(y.cpu().numpy(), want, "attention prefill")
    assert_close(attn.k_cache[:, :, :S].cpu().numpy(), oattn.k_cache[:, :, :S], 1e-2, 4e-3, "k cache after the prompt")
    z = ffn.forward(y, True, True)
    close(z.cpu().numpy(), offn.forward(y.cpu().numpy()), "ffn prefill")
    x1 = torch.randn(B, 1, cfg.hidden, generator=g).half()
    y = attn.forward(x1.to(gpu), e, e, True, True, False, torch.empty(0))
    want = oattn.forward(x1.numpy(), None, False, None)
    close(y.cpu().numpy(), want, "attention step 1025")
    del model
    ops.workspaces.clear()
    torch.cuda.empty_cache()
