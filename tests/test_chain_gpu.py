"""Chained launches (eet_gemm_w8a16_chained): kernels enqueued without the queue barrier that wait
in the kernel for their producer's completion counter.  Every launch of a chain reads what the
previous one wrote, so a consumer that ran ahead of its producer, or read a stale cache line,
shows as a mismatch.  Results must be bit-identical to the ordinary launches
(eet_gemm_w8a16_fused) and within the GEMM tolerance of the oracle; the bounded wait is made to
give up from the host (spin limit 0) and must report it while every kernel still exits."""
import ctypes

import numpy as np
import pytest
import torch

from eet_amd import ops
from eet_amd._lib import check, lib
from oracle import ops as O

from gpu_util import assert_close, gemm_fused, stream

pytestmark = pytest.mark.gpu

NONE, RES, SWIGLU = 0, 1, 2
FIRST, NEXT = 1, 2


def make_linear(K, N, seed, gpu):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(K, N, generator=g) * 0.02).half()
    u, p, s = ops.quant_weights(w, torch.int8, True)
    return u, s, p.to(gpu), s.to(gpu)


def chained(a, wp, s, c, M, N, K, epi, residual, gamma, eps, mode):
    check(lib().eet_gemm_w8a16_chained(a.data_ptr(), wp.data_ptr(), s.data_ptr(), c.data_ptr(), M, N, K, epi,
                                       residual.data_ptr() if residual is not None else None,
                                       gamma.data_ptr() if gamma is not None else None, eps, mode, stream()),
          "eet_gemm_w8a16_chained")


def chain_status(clear=True):
    flag = ctypes.c_int(-1)
    check(lib().eet_chain_status(ctypes.byref(flag), 1 if clear else 0, stream()), "eet_chain_status")
    return flag.value


def layer_launches(hidden, d_ff, gpu, seed):
    """The four int8 launches of a decoder layer with a real data flow between them:
    h0 -> RMSnorm + gate|up + SwiGLU -> act -> down + h0 -> h1 -> O-shaped + h1 -> h2 -> RMSnorm + QKV -> qkv."""
    gu, gs, gp, gsd = make_linear(hidden, d_ff, seed, gpu)
    uu, us, up, usd = make_linear(hidden, d_ff, seed + 1, gpu)
    w01, s01 = ops.interleave_gate_up(gp, gsd, up, usd)
    down = make_linear(d_ff, hidden, seed + 2, gpu)
    o = make_linear(hidden, hidden, seed + 3, gpu)
    qkv = make_linear(hidden, 3 * hidden, seed + 4, gpu)
    g = torch.Generator().manual_seed(seed + 5)
    gam1 = (1 + 0.1 * torch.randn(hidden, generator=g)).half().to(gpu)
    gam2 = (1 + 0.1 * torch.randn(hidden, generator=g)).half().to(gpu)
    return dict(w01=w01, s01=s01, down=down, o=o, qkv=qkv, gam1=gam1, gam2=gam2, gate=(gu, gs), up=(uu, us))


def run_layer(L, bufs, M, hidden, d_ff, launch):
    """launch(a, wp, s, c, M, N, K, epi, residual, gamma) issues one GEMM."""
    launch(bufs["h0"], L["w01"], L["s01"], bufs["act"], M, 2 * d_ff, hidden, SWIGLU, None, L["gam1"])
    launch(bufs["act"], L["down"][2], L["down"][3], bufs["h1"], M, hidden, d_ff, RES, bufs["h0"], None)
    launch(bufs["h1"], L["o"][2], L["o"][3], bufs["h2"], M, hidden, hidden, RES, bufs["h1"], None)
    launch(bufs["h2"], L["qkv"][2], L["qkv"][3], bufs["qkv"], M, 3 * hidden, hidden, NONE, None, L["gam2"])


@pytest.mark.parametrize("hidden,d_ff,M", [(4096, 11008, 8), (4096, 11008, 1), (4096, 11008, 16),
                                           (5120, 13696, 32), (5120, 13696, 8), (256, 704, 5)])
def test_chained_layer_matches_ordinary_launches(gpu, hidden, d_ff, M):
    L = layer_launches(hidden, d_ff, gpu, seed=hidden + M)
    g = torch.Generator().manual_seed(M)

    def buffers():
        return {"h0": None, "act": torch.zeros(M, d_ff, dtype=torch.float16, device=gpu),
                "h1": torch.zeros(M, hidden, dtype=torch.float16, device=gpu),
                "h2": torch.zeros(M, hidden, dtype=torch.float16, device=gpu),
                "qkv": torch.zeros(M, 3 * hidden, dtype=torch.float16, device=gpu)}
    eps = 1e-6
    inputs = [torch.randn(M, hidden, generator=g).half().to(gpu) for _ in range(6)]

    def plain(a, wp, s, c, M_, N, K, epi, residual, gamma):
        check(lib().eet_gemm_w8a16_fused(a.data_ptr(), wp.data_ptr(), s.data_ptr(), c.data_ptr(), M_, N, K, epi,
                                         residual.data_ptr() if residual is not None else None,
                                         gamma.data_ptr() if gamma is not None else None, eps, None, 0, stream()))
    # ordinary launches, one input after the other; act, h1, h2 are reused by every input, each input
    # has its own qkv rows (which depend on every launch before them)
    b = buffers()
    want_qkv = []
    for x in inputs:
        b["h0"], b["qkv"] = x, torch.zeros(M, 3 * hidden, dtype=torch.float16, device=gpu)
        run_layer(L, b, M, hidden, d_ff, plain)
        want_qkv.append(b["qkv"])
    want_last = {k: b[k].clone() for k in ("act", "h1", "h2")}
    first_act = None
    torch.cuda.synchronize()
    # the same as ONE chain of 24 launches with nothing else enqueued in between: a launch that ran ahead
    # of its producer would read the previous input's values from the shared buffers
    print(f"chained layer: hidden={hidden} d_ff={d_ff} M={M}", flush=True)
    assert chain_status() == 0
    b = buffers()
    got_qkv = [torch.zeros(M, 3 * hidden, dtype=torch.float16, device=gpu) for _ in inputs]
    first = [True]

    def link(a, wp, s, c, M_, N, K, epi, residual, gamma):
        chained(a, wp, s, c, M_, N, K, epi, residual, gamma, eps, FIRST if first[0] else NEXT)
        first[0] = False
    for x, q in zip(inputs, got_qkv):
        b["h0"], b["qkv"] = x, q
        run_layer(L, b, M, hidden, d_ff, link)
    assert chain_status() == 0, "a chained wait gave up"      # waits for the stream
    for i, (gq, wq) in enumerate(zip(got_qkv, want_qkv)):
        assert torch.equal(gq, wq), (i, float((gq.float() - wq.float()).abs().max()))
    for k, w in want_last.items():
        assert torch.equal(b[k], w), k
    # a new chain (its first launch is an ordinary one, ordered behind the reads above) for the first input alone
    got = [{}]
    b["h0"] = inputs[0]
    first[0] = True
    run_layer(L, b, M, hidden, d_ff, link)
    assert chain_status() == 0
    got[0]["act"] = b["act"]
    assert torch.equal(b["qkv"], want_qkv[0])
    # and against the oracle for the first launch of the first input (gate|up + SwiGLU with the RMSnorm prologue)
    if hidden <= 4096:
        x = inputs[0].cpu().numpy()
        xn = O.rmsnorm(x, L["gam1"].cpu().numpy(), eps)
        gate = O.dequant_matmul(xn, L["gate"][0].numpy(), L["gate"][1].numpy(), np.float16)
        upv = O.dequant_matmul(xn, L["up"][0].numpy(), L["up"][1].numpy(), np.float16)
        ref = O.swiglu(gate, upv)
        assert_close(got[0]["act"].float().cpu().numpy(), ref.astype(np.float32), atol=3e-3, what="chained gate|up+SwiGLU")


def test_chain_long_run_stays_ordered(gpu):
    """A few hundred chained launches in a row where each launch consumes the previous one's output (a
    square GEMM with the residual epilogue feeding itself through two buffers), against the ordinary
    launches: any launch that overtook its producer changes every later value."""
    hidden, M = 4096, 8
    _, _, wp, sd = make_linear(hidden, hidden, 77, gpu)
    sd = (sd.float() * 0.02).half()          # x <- x + W.x with a small W: the values stay in range for 300 steps
    x0 = (torch.randn(M, hidden, generator=torch.Generator().manual_seed(5)) * 0.5).half().to(gpu)
    eps = 0.0

    def run(launch, n):
        bufs = [x0.clone(), torch.zeros_like(x0)]
        for i in range(n):
            a, c = bufs[i % 2], bufs[(i + 1) % 2]
            launch(a, c, i)
        return bufs[n % 2].clone()
    n = 300
    want = run(lambda a, c, i: check(lib().eet_gemm_w8a16_fused(
        a.data_ptr(), wp.data_ptr(), sd.data_ptr(), c.data_ptr(), M, hidden, hidden, RES, a.data_ptr(), None, eps, None,
        0, stream())), n)
    torch.cuda.synchronize()
    print("chained long run: 300 dependent launches", flush=True)
    got = run(lambda a, c, i: chained(a, wp, sd, c, M, hidden, hidden, RES, a, None, eps, FIRST if i == 0 else NEXT), n)
    assert chain_status() == 0
    assert torch.isfinite(want.float()).all()
    assert torch.equal(got, want)


def test_chain_argument_errors(gpu):
    _, _, wp, sd = make_linear(256, 256, 3, gpu)
    a = torch.zeros(64, 256, dtype=torch.float16, device=gpu)
    c = torch.zeros(64, 256, dtype=torch.float16, device=gpu)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        # nothing chained on this stream yet
        with pytest.raises(RuntimeError, match="previous chained launch on the same stream"):
            chained(a, wp, sd, c, 8, 256, 256, NONE, None, None, 0.0, NEXT)
    with pytest.raises(RuntimeError, match="M <= 32"):
        chained(a, wp, sd, c, 64, 256, 256, NONE, None, None, 0.0, FIRST)
    with pytest.raises(RuntimeError, match="unknown chain mode"):
        chained(a, wp, sd, c, 8, 256, 256, NONE, None, None, 0.0, 7)
    # refused while the stream records a graph (the first launch of a chain is an ordinary one and may be recorded)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="HIP graph"):
        with torch.cuda.graph(g):
            chained(a, wp, sd, c, 8, 256, 256, NONE, None, None, 0.0, FIRST)
            chained(a, wp, sd, c, 8, 256, 256, NONE, None, None, 0.0, NEXT)
    torch.cuda.synchronize()


def test_bounded_wait_gives_up_and_reports(gpu, tuning):
    """Spin limit 0: a chained consumer gives up without polling.  Every kernel still exits (the
    synchronisation returns), the error word is set, and clearing it restores a clean status."""
    _, _, wp, sd = make_linear(1024, 1024, 9, gpu)
    a = torch.randn(8, 1024, generator=torch.Generator().manual_seed(1)).half().to(gpu)
    c1, c2 = torch.zeros_like(a), torch.zeros_like(a)
    assert chain_status() == 0
    tuning("EET_CHAIN_SPIN_LIMIT", 0)
    print("bounded wait: spin limit 0", flush=True)
    chained(a, wp, sd, c1, 8, 1024, 1024, NONE, None, None, 0.0, FIRST)
    chained(c1, wp, sd, c2, 8, 1024, 1024, NONE, None, None, 0.0, NEXT)
    assert chain_status(clear=False) == 1          # waits for the stream: both kernels have exited
    assert chain_status(clear=True) == 1
    assert chain_status() == 0
    lib().eet_set_tuning(b"EET_CHAIN_SPIN_LIMIT", None)
    chained(a, wp, sd, c1, 8, 1024, 1024, NONE, None, None, 0.0, FIRST)
    chained(c1, wp, sd, c2, 8, 1024, 1024, NONE, None, None, 0.0, NEXT)
    assert chain_status() == 0
    want = gemm_fused(gemm_fused(a, wp, sd, 8, 1024, 1024, NONE), wp, sd, 8, 1024, 1024, NONE)
    torch.cuda.synchronize()
    assert torch.equal(c2, want)
