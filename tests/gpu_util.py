"""Helpers shared by the GPU parity tests: calls go through the C ABI."""
import numpy as np
import torch

from eet_amd._lib import check, lib

# north-star tolerance against the fp32 oracle: 1e-2 relative / 1e-3 absolute
RTOL, ATOL = 1e-2, 1e-3


def stream():
    return torch.cuda.current_stream().cuda_stream


def assert_close(got, want, rtol=RTOL, atol=ATOL, what=""):
    got = np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    tol = atol + rtol * np.abs(want)
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} outside tolerance, max err {err.max():.5f}"


def gemm(a, wp, s, M, N, K):
    c = torch.empty(M, N, dtype=torch.float16, device=a.device)
    check(lib().eet_gemm_w8a16(a.data_ptr(), wp.data_ptr(), s.data_ptr(), c.data_ptr(), M, N, K, None, 0, stream()),
          "eet_gemm_w8a16")
    return c


def mmha(q, k, v, kc, vc, step, pad=None, alibi=None, stride=0, rope_row=None):
    B, H, T, dh = kc.shape
    ctx = torch.empty(B, H * dh, dtype=torch.float16, device=kc.device)
    L = lib()
    need = L.eet_mmha_decode_workspace(B, H, dh, step)
    ws = torch.empty(max(need // 4, 1), dtype=torch.float32, device=kc.device)
    check(L.eet_mmha_decode(q.data_ptr(), k.data_ptr() if k is not None else None,
                            v.data_ptr() if v is not None else None, stride, kc.data_ptr(), vc.data_ptr(),
                            ctx.data_ptr(), alibi.data_ptr() if alibi is not None else None,
                            pad.data_ptr() if pad is not None else None, B, H, dh, step, T,
                            rope_row.data_ptr() if rope_row is not None else None, ws.data_ptr(),
                            ws.numel() * 4, stream()), "eet_mmha_decode")
    return ctx
