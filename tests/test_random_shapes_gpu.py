"""Seeded random shapes through the C ABI against the fp32 oracle: the fused dequant-GEMM over every
dispatch range (small-M, 32-row slabs, every large-M tile) with each epilogue and the RMSnorm prologue,
and the decode attention over random batch / head / step / padding / ALiBi combinations.
Tolerance: 1e-2 relative / 1e-3 absolute (2e-3 / 3e-3 absolute with the RMSnorm prologue / + SwiGLU,
whose reference composition rounds once more), as in the per-kernel tests."""
import numpy as np
import pytest
import torch

import eet_amd
from eet_amd.ops import interleave_gate_up
from oracle import ops as O

from gpu_util import assert_close, gemm, gemm_fused as _fused, mmha

pytestmark = pytest.mark.gpu


def _gemm_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        m_hi = [8, 32, 128, 700][i % 4]                       # small-M, small-M with 2-4 row groups, slabs, large-M
        M = int(rng.integers(1, m_hi + 1))
        K = 64 * int(rng.integers(1, 24))
        N = 16 * int(rng.integers(1, 70))
        epi = int(rng.integers(0, 3))
        if epi == 2:
            N = max(32, N // 32 * 32)
        rms = bool(rng.integers(0, 2)) and M <= 32
        cases.append((M, K, N, epi, rms, int(rng.integers(1 << 30))))
    return cases


@pytest.mark.parametrize("M,K,N,epi,rms,seed", _gemm_cases(48, 2024))
def test_gemm_random(gpu, M, K, N, epi, rms, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(M, K, generator=g) * 1.3).half()
    gamma = (1 + 0.1 * torch.randn(K, generator=g)).half() if rms else None
    eps = 1e-6
    x32 = x.numpy().astype(np.float32)
    if rms:   # un-rounded composition: the kernel rounds x * gamma once and scales the fp32 sum by 1 / rms
        xin = x32 * gamma.numpy().astype(np.float32) / np.sqrt((x32 * x32).mean(1, keepdims=True) + eps)
    else:
        xin = x32
    if epi == 2:
        F = N // 2
        wg = (torch.randn(K, F, generator=g) * 0.02).half()
        wu = (torch.randn(K, F, generator=g) * 0.02).half()
        ug, pg, sg = eet_amd.quant_weights(wg, torch.int8, True)
        uu, pu, su = eet_amd.quant_weights(wu, torch.int8, True)
        wp, s = interleave_gate_up(pg, sg, pu, su)
        want = O.swiglu(O.dequant_matmul(xin, ug.numpy(), sg.numpy(), np.float32).astype(np.float16),
                        O.dequant_matmul(xin, uu.numpy(), su.numpy(), np.float32).astype(np.float16))
        res = None
    else:
        w = (torch.randn(K, N, generator=g) * 0.02).half()
        u, wp, s = eet_amd.quant_weights(w, torch.int8, True)
        want = O.dequant_matmul(xin, u.numpy(), s.numpy(), np.float32)
        res = torch.randn(M, N, generator=g).half() if epi == 1 else None
        if epi == 1:
            want = O.residual_add(want.astype(np.float16), res.numpy())
    got = _fused(x.to(gpu), wp.to(gpu), s.to(gpu), M, N, K, epi, res.to(gpu) if res is not None else None,
                 gamma.to(gpu) if rms else None, eps).cpu().numpy()
    atol = (3e-3 if epi == 2 else 2e-3) if (rms or epi == 1) else 1e-3
    assert_close(got, want, rtol=1e-2, atol=atol, what=f"M={M} K={K} N={N} epi={epi} rms={rms}")
    if epi == 0 and not rms:   # the plain entry point takes the same path
        assert torch.equal(gemm(x.to(gpu), wp.to(gpu), s.to(gpu), M, N, K).cpu(), torch.from_numpy(got))


def _attn_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        dh = [32, 64, 96, 128][int(rng.integers(0, 4))]
        B, H = int(rng.integers(1, 6)), int(rng.integers(1, 9))
        step = int(rng.integers(1, [40, 400, 1500, 4000][i % 4]))
        cases.append((B, H, dh, step, step + int(rng.integers(0, 9)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2)),
                      int(rng.integers(1 << 30))))
    return cases


@pytest.mark.parametrize("B,H,dh,step,cap,use_pad,use_alibi,seed", _attn_cases(24, 77))
def test_attention_random(gpu, B, H, dh, step, cap, use_pad, use_alibi, seed):
    g = torch.Generator().manual_seed(seed)
    kc = torch.randn(B, H, cap, dh, generator=g).half()
    vc = torch.randn(B, H, cap, dh, generator=g).half()
    q, k, v = [torch.randn(B, H, dh, generator=g).half() for _ in range(3)]
    pad = torch.randint(0, step + 1, (B,), generator=g) if use_pad else None   # may pad a whole sequence away
    alibi = torch.from_numpy(O.alibi_bias(H, step)) if use_alibi else None
    kcn, vcn = kc.numpy().copy(), vc.numpy().copy()
    want = O.decode_attention(q.numpy(), k.numpy(), v.numpy(), kcn, vcn, step, pad.numpy() if use_pad else None,
                              alibi.numpy() if use_alibi else None)
    kcd, vcd = kc.to(gpu), vc.to(gpu)
    ctx = mmha(q.to(gpu), k.to(gpu), v.to(gpu), kcd, vcd, step, pad.to(gpu) if use_pad else None,
               alibi.to(gpu) if use_alibi else None)
    assert_close(ctx.cpu().numpy(), want, what=f"B={B} H={H} dh={dh} step={step} pad={use_pad} alibi={use_alibi}")
    assert np.array_equal(kcd.cpu().numpy(), kcn) and np.array_equal(vcd.cpu().numpy(), vcn)


def _prefill_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        dh = [128, 128, 64, 128, 96, 128, 32, 128][i % 8]          # mostly the DMA kernel (head size 128)
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
        S = int(rng.integers(1, [70, 300, 600, 1100][i % 4]))
        cases.append((B, H, dh, S, S + int(rng.integers(0, 9)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2)),
                      int(rng.integers(1 << 30))))
    return cases


@pytest.mark.parametrize("B,H,dh,S,cap,use_pad,use_alibi,seed", _prefill_cases(24, 99))
def test_prefill_attention_random(gpu, B, H, dh, S, cap, use_pad, use_alibi, seed):
    """Causal prompt attention over random batch / head / length / padding / ALiBi combinations (odd lengths,
    lengths around the 64-key chunk and 256-query block edges, a padding that covers a whole prompt)."""
    from eet_amd._lib import check, lib
    from gpu_util import stream
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(B, H, S, dh, generator=g).half() for _ in range(3)]
    kc = torch.randn(B, H, cap, dh, generator=g).half()          # rows past S hold junk that must not be read
    vc = torch.randn(B, H, cap, dh, generator=g).half()
    kc[:, :, :S], vc[:, :, :S] = k, v
    pad = torch.randint(0, S + 1, (B,), generator=g) if use_pad else None
    want = O.prefill_attention(q.numpy(), k.numpy(), v.numpy(), pad.numpy() if use_pad else None,
                               O.alibi_mask(H, S) if use_alibi else None)
    ctx = torch.full((B, S, H * dh), float("nan"), dtype=torch.float16, device=gpu)
    row = torch.from_numpy(O.alibi_bias(H, S)).to(gpu) if use_alibi else None
    padd = pad.to(gpu) if use_pad else None
    qd, kcd, vcd = q.to(gpu), kc.to(gpu), vc.to(gpu)
    check(lib().eet_prefill_attention(qd.data_ptr(), kcd.data_ptr(), vcd.data_ptr(), ctx.data_ptr(),
                                      row.data_ptr() if use_alibi else None, padd.data_ptr() if use_pad else None,
                                      B, H, S, dh, cap, stream()))
    assert_close(ctx.cpu().numpy(), want, what=f"B={B} H={H} dh={dh} S={S} pad={use_pad} alibi={use_alibi}")
