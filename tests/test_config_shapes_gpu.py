"""GPU parity at the full shapes of benchmark configurations 3 and 5 (Baichuan-13B: hidden 5120,
intermediate 13696), against the fp32 oracle, through the C ABI.

Configuration 3: the prefill GEMMs at M = 2048 (QKV 5120 -> 15360, O 5120 -> 5120, gate / up
5120 -> 13696, down 13696 -> 5120), i.e. the 128 x 256 and 64 x 320 MFMA tiles the dispatcher
picks there, every output element compared.
Configuration 5: the decode linears at M = 32 as the decoder ops launch them (RMSnorm prologue on
QKV and gate|up, SwiGLU epilogue, residual epilogue on O and down).
Tolerance: 1e-2 relative / 1e-3 absolute against dequantise-then-matmul in fp32; the fused decode
launches are held to per-launch absolute bounds of 1.5 x their measured need (BOUNDS below)."""
import numpy as np
import pytest
import torch

import eet_amd
from oracle import ops as O

from gpu_util import assert_close, gemm, gemm_fused, measured

pytestmark = pytest.mark.gpu

HIDDEN, DFF = 5120, 13696


def weights(K, N, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(K, N, generator=g) * 0.02).half()
    u, p, s = eet_amd.quant_weights(w, torch.int8, True)
    return u, p, s


@pytest.mark.parametrize("name,K,N", [("qkv", HIDDEN, 3 * HIDDEN), ("o", HIDDEN, HIDDEN), ("gate", HIDDEN, DFF),
                                      ("down", DFF, HIDDEN)])
def test_config3_prefill_gemm(gpu, name, K, N):
    M = 2048
    u, p, s = weights(K, N, K + N)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(N)).half()
    print(f"config 3 {name}: M={M} K={K} N={N}", flush=True)
    c = gemm(x.to(gpu), p.to(gpu), s.to(gpu), M, N, K).cpu().numpy()
    want = O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32)
    assert_close(c, want, what=f"config 3 {name}")


def test_config3_gate_up_swiglu(gpu):
    """gate and up in one launch with the SwiGLU epilogue at M = 2048 (what the FFN op launches for a prompt)."""
    from eet_amd.ops import interleave_gate_up
    M, K, F = 2048, HIDDEN, DFF
    ug, pg, sg = weights(K, F, 1)
    uu, pu, su = weights(K, F, 2)
    w01, s01 = interleave_gate_up(pg, sg, pu, su)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(3)).half()
    print(f"config 3 gate|up+swiglu: M={M} K={K} N={2 * F}", flush=True)
    got = gemm_fused(x.to(gpu), w01.to(gpu), s01.to(gpu), M, 2 * F, K, 2).cpu().numpy()
    want = O.swiglu(O.dequant_matmul(x.numpy(), ug.numpy(), sg.numpy()),
                    O.dequant_matmul(x.numpy(), uu.numpy(), su.numpy()))
    assert_close(got, want, rtol=1e-2, atol=1e-3, what="config 3 gate|up")


# Absolute tolerance each fused launch may need at 1e-2 relative: 1.5 x the need observed on an MI355X
# (in brackets), and the north-star's 1e-3 wherever the observed need is below it.  Only the launches
# that compare against a composition with NO intermediate fp16 rounding need more: the RMSnorm prologue
# rounds x * gamma where the unfused path rounds x * gamma / rms, and the SwiGLU epilogue rounds gate and
# up to fp16 (as the separate GEMMs would) before multiplying them.
BOUNDS = {("qkv", 32): 1.6e-3,      # [1.06e-3]
          ("qkv", 8): 1e-3,         # [9.7e-4]
          ("o", 32): 1e-3,          # [5.9e-4]
          ("o", 8): 1e-3,           # [2.8e-5]
          ("gate|up", 32): 4.4e-3,  # [2.93e-3]
          ("gate|up", 8): 3.2e-3,   # [2.11e-3]
          ("down", 32): 1e-3,       # [9.8e-5]
          ("down", 8): 1e-3}        # [6.5e-4]


def _rms_f32(x, gamma, eps):
    x32 = x.numpy().astype(np.float32)
    return x32 / np.sqrt((x32 * x32).mean(-1, keepdims=True) + np.float32(eps)) * gamma.numpy().astype(np.float32)


@pytest.mark.parametrize("M", [32, 8])
def test_config5_decode_linears(gpu, M):
    """The four launches of a Baichuan-13B decoder layer at batch 32 (and 8), with their fused parts.
    The RMSnorm prologue is compared with the composition without an intermediate rounding; the error of
    every launch is printed and held to the per-launch bound of BOUNDS at 1e-2 relative."""
    from eet_amd.ops import interleave_gate_up
    g = torch.Generator().manual_seed(50 + M)
    eps = 1e-6
    x = (torch.randn(M, HIDDEN, generator=g) * 1.3).half()
    gamma = (1 + 0.1 * torch.randn(HIDDEN, generator=g)).half()
    xn = _rms_f32(x, gamma, eps)
    xd, gd = x.to(gpu), gamma.to(gpu)

    # QKV with the RMSnorm prologue: 5120 -> 15360
    u, p, s = weights(HIDDEN, 3 * HIDDEN, 5)
    print(f"config 5 qkv+rmsnorm M={M}", flush=True)
    got = gemm_fused(xd, p.to(gpu), s.to(gpu), M, 3 * HIDDEN, HIDDEN, 0, None, gd, eps).cpu().numpy()
    want = xn @ (u.numpy().astype(np.float32) * s.numpy().astype(np.float32)[None, :])
    measured(got, want, f"config5 rmsnorm+qkv M={M}", BOUNDS.get(("qkv", M)))

    # O + residual: 5120 -> 5120
    u, p, s = weights(HIDDEN, HIDDEN, 6)
    ctx = torch.randn(M, HIDDEN, generator=g).half()
    print(f"config 5 o+residual M={M}", flush=True)
    got = gemm_fused(ctx.to(gpu), p.to(gpu), s.to(gpu), M, HIDDEN, HIDDEN, 1, xd).cpu().numpy()
    want = O.residual_add(O.dequant_matmul(ctx.numpy(), u.numpy(), s.numpy()), x.numpy())
    measured(got, want, f"config5 o+residual M={M}", BOUNDS.get(("o", M)))

    # gate|up with the RMSnorm prologue and the SwiGLU epilogue: 5120 -> 27392
    ug, pg, sg = weights(HIDDEN, DFF, 7)
    uu, pu, su = weights(HIDDEN, DFF, 8)
    w01, s01 = interleave_gate_up(pg, sg, pu, su)
    print(f"config 5 gate|up+rmsnorm+swiglu M={M}", flush=True)
    got = gemm_fused(xd, w01.to(gpu), s01.to(gpu), M, 2 * DFF, HIDDEN, 2, None, gd, eps).cpu().numpy()
    gate = xn @ (ug.numpy().astype(np.float32) * sg.numpy().astype(np.float32)[None, :])
    up = xn @ (uu.numpy().astype(np.float32) * su.numpy().astype(np.float32)[None, :])
    measured(got, up * gate / (1 + np.exp(-gate)), f"config5 rmsnorm+gate|up+swiglu M={M}", BOUNDS.get(("gate|up", M)))

    # down + residual: 13696 -> 5120
    u, p, s = weights(DFF, HIDDEN, 9)
    act = (torch.randn(M, DFF, generator=g) * 0.5).half()
    print(f"config 5 down+residual M={M}", flush=True)
    got = gemm_fused(act.to(gpu), p.to(gpu), s.to(gpu), M, HIDDEN, DFF, 1, xd).cpu().numpy()
    want = O.residual_add(O.dequant_matmul(act.numpy(), u.numpy(), s.numpy()), x.numpy())
    measured(got, want, f"config5 down+residual M={M}", BOUNDS.get(("down", M)))
